"""Per-GPU rendezvous of the K virtual stream workers (VSWs) around one fused launch.

In IIDP every VSW runs its own DDP reducer on its own thread and stream; only VSW 0's
comm hook communicates, the others register ``dummy_hook``
(jabas/train/trainer.py:452-468). ``LocalBucketSync`` is where those K hooks meet on one
GPU: each hook publishes the flat bucket it was handed; when the K buckets with the same
index are in, whichever thread arrived last queues ONE fused kernel (aggregate into VSW 0's
bucket, statistics when asked, optimizer update and weight fan-out when an optimizer is
bound). The Future a hook gets back is already complete: stock DDP waits on it at the end
of that replica's backward on the autograd engine's device thread, which every replica on
the GPU shares, so a Future that needed another replica's backward to make progress would
deadlock. Ordering is by stream instead: the launch waits on an event from every VSW's
stream, and ``finish_step`` makes every VSW stream wait for the launches (and reports
anything that went wrong in them) before gradients and weights are reused. The step ends by
itself with the hand-over that completes the replicas' last bucket (``GradBucket.is_last()``),
so a loop that only registers the hooks calls nothing else.

Hooks that carry no state of ours (the reference registers ``dummy_hook`` with ``state=None``
and builds the main state without any handle to IIDP's local machinery) find the object through
the device it was installed for (``install``) and their VSW index through the replica a bucket's
parameters belong to (``register_replicas``) or the stream they run on.

The "overlap" weight-sync mode (jabas/train/trainer.py:327-333: an optimizer hook on VSW 0
that updates the weights of a bucket as soon as its gradients are synchronised, on a stream
of its own) is this class with an optimizer bound (``bind_optimizer``) and a launch stream
(``stream=``): the weights and optimizer state of a bucket's parameters are laid out in
flat arenas exactly like the bucket, so aggregate, update and the copy of the new weights
to the other replicas are one launch per bucket.
"""
import ctypes as C
import threading
import weakref

import torch

from . import sync
from . import _lib as L

# The meeting point of each device, for hooks that are registered without a state of ours: the reference
# registers ``dummy_hook`` with ``state=None`` on every VSW but the first and builds the main VSW's state
# without any handle to IIDP's local machinery (jabas/train/trainer.py:452-468), so both find the GPU's
# LocalBucketSync here. Filled by ``LocalBucketSync.install`` (what stands in for IIDP's trainer calls it
# when it builds the local models); weak references: an object nobody holds any more is not found.
_installed = {}
_installed_lock = threading.Lock()


def _device_key(device):
    if device is None:
        return "cpu"
    device = torch.device(device)
    if device.type != "cuda":
        return "cpu"
    return device.index if device.index is not None else torch.cuda.current_device()


def installed(device):
    """The LocalBucketSync installed for ``device`` (a torch.device, or None for host tensors), or None."""
    ref = _installed.get(_device_key(device))
    return None if ref is None else ref()


class BucketStats:
    """Statistics row of one bucket on the device (what a stat step leaves in
    ``GradientSimilarityState.grad_placeholder`` instead of a full gradient copy). The row is
    one of two buffers the bucket's launches alternate between: read it (``cpu()``) before the
    second-next statistic step of that bucket."""

    def __init__(self, index, row):
        self.index, self.row = index, row

    def cpu(self):
        return self.row.detach().to("cpu")


class _Slot:
    def __init__(self, K):
        self.tensors = [None] * K
        self.buckets = [None] * K
        self.events = [None] * K
        self.want_stats = False
        self.on_done = None
        self.count = 0


def _arena_like(buf, dtype=torch.float32, zero=True):
    """Flat tensor of ``buf.numel()`` elements of ``dtype`` whose first element sits at the same element
    position of a 256-byte line as ``buf``'s (the layout the kernels stream fastest, and the congruence
    they require)."""
    n = buf.numel()
    raw = (torch.zeros if zero else torch.empty)(n + 64, dtype=dtype, device=buf.device)
    want = (buf.data_ptr() // buf.element_size()) % 64
    have = (raw.data_ptr() // raw.element_size()) % 64
    return raw[(want - have) % 64:][:n]


class LocalBucketSync:
    """batches: local batch size of each VSW on this GPU (defines K and the weights).

    launcher(bucket_index, tensors, want_stats) -> stats row or None replaces the C-ABI
    call (CPU tests of the protocol inject a recorder); the default queues
    ``jabas_sync_bucket`` on the launch stream.
    """

    def __init__(self, batches, launcher=None, opt=None, param_buckets=None, deferred=False, stream=None,
                 optimizer=None, stats_level="similarity", batch_bytes=0, share_weights=False, write_aggregate=True,
                 launch_streams=2, auto_finish=True, interleave_moments=False, launch_on_last_vsw=False):
        """deferred: collect the buckets of a step and queue ONE planned launch over all of them in
        ``finish_step`` instead of one launch per bucket as each becomes complete. The per-bucket mode
        overlaps the sync with the rest of the backward pass; the deferred mode spends less GPU time
        (one ramp-up and drain: 0.68 ms against 0.9 ms wall for the 14 buckets of ViT-B/16) and less host
        time, and the buckets hold the aggregate only after ``finish_step``.

        batch_bytes: between the two: complete buckets are held back until this many bytes of them (size of
        one VSW's buffers) are ready, then go out as ONE planned launch behind one event wait per VSW
        (what remains at the end of the step goes out in ``finish_step``). The sync still overlaps the
        backward passes, in coarser steps; every launch costs the host K stream waits and the GPU a ramp-up
        and drain, which is what batching divides (14 x 25 MB buckets of ViT-B/16 in batches of 64 MB: five
        launches instead of fourteen). 0: one launch per bucket.

        stats_level: what a statistic step computes per bucket: "similarity" (the four sums the cosine between
        the halves and norm clipping read: all the reference's adaptive batching consumes,
        jabas/train/trainer.py:470-483), "full" (plus the squared norm of every VSW's gradient) or "gram" (plus
        the product of every pair of VSWs' gradients, the worker x worker Gram matrix, out of the same launch:
        up to eight VSWs; ``sync.gram_from_stats`` reads it from the rows).

        stream: the stream the fused launches are queued on (the reference's dedicated optimizer
        stream, jabas/train/trainer.py:328); default: the stream VSW 0's hooks run on.

        launch_streams (with ``stream=``): how many launch streams the buckets' launches alternate between
        (bucket i goes to stream i mod launch_streams; the first is ``stream``, the others are made here at the
        default priority). Consecutive buckets are independent of each other, so on two streams the last
        workgroups of one bucket's launch drain while the next bucket's launch is already filling the chip,
        instead of one launch waiting for the one before to finish to the last wave (measured on the ViT-L/16 set,
        38 buckets: 2.61 ms a step on one stream, 6 us of idle queue between launches, 2.37 ms on two, which is
        what one launch over all buckets takes; a third stream gains nothing). ``finish_step`` orders the VSW
        streams behind every one of them.

        launch_on_last_vsw (without ``stream=``): a bucket's launch goes on the stream of the VSW whose hand-over
        completed the bucket, behind an event from every other VSW's stream, instead of on VSW 0's stream or on
        launch streams of its own. No stream beyond the K the VSWs run on is needed (a GPU serves a process
        through a handful of hardware queues; streams beyond them share one and run in submission order, which
        launch streams on top of three or more VSW streams run into), consecutive buckets completed by
        different VSWs still overlap their ramp-up and drain, and the VSW that came last finds the launch ahead
        of the rest of its own backward pass, which nobody else waits for.

        auto_finish: when the bucket objects tell which bucket is a replica's last (``GradBucket.is_last()``),
        the hand-over that completes that bucket also ends the step (``finish_step`` with the streams the hooks
        ran on), so a training loop that only registers the hooks needs no call of its own; a later
        ``finish_step()`` of the same step is then a no-op (it still orders the streams it is given behind the
        step's launches).

        share_weights (with ``optimizer=``): the parameters of the other VSWs' models become views of the main
        model's weight arena instead of arenas of their own that every launch refreshes. The VSWs of a GPU hold
        identical weights after every step and a bucket is updated only once every VSW is past its parameters
        in the backward pass, so one copy serves all: 4 (K - 1) fewer bytes written per element and step, K - 1
        fewer copies of the weights in HBM. The replicas take the main model's values when a bucket is bound.

        write_aggregate=False (buckets whose launch runs the optimizer only): the aggregate goes to the update
        in registers and is written nowhere, neither into VSW 0's fp32 bucket nor into an fp32 arena beside a
        reduced-precision one: 4 bytes per element fewer. For callers that read no gradient after the step; the
        default leaves the synchronised gradient in the main VSW's bucket, as the reference's hooks do. Buckets
        under a norm bound (``grad_clip``) keep the write: their second launch reads the aggregate.

        interleave_moments (with ``optimizer=``, Adam kinds): the moments of a bucket's parameters are kept in
        one arena of alternating blocks (``sync.MomentArena``: the layout the kernels stream 2-6 % faster) instead
        of flat arenas. A moment then is no flat tensor: the optimizer object gets copies under torch's names
        when its ``state_dict()`` runs (hooks on the optimizer) and holds only the step count in between; state
        the optimizer carries in when a bucket is bound (a checkpoint loaded before the first step) is taken
        over. Default: flat arenas whose views ``optimizer.state[p]`` holds at all times.

        opt + param_buckets: hyperparameter dictionary and, per bucket index, dict(param=, state1=,
        state2=, state3=, bounds=, fanout=, agg_out=) of flat fp32 tensors laid out like the bucket (or, in place of
        the state tensors of an Adam kind, moments=(sync.MomentArena, index of the bucket's first element in it):
        the moments interleaved in one arena, the layout the kernels stream fastest); the launch of
        such a bucket also runs the optimizer. ``optimizer=`` (or ``bind_optimizer``) takes a
        torch.optim.SGD / Adam / AdamW or Shard* object instead and builds those arenas itself from the
        ``parameters()`` / ``gradients()`` of the bucket objects the hooks publish."""
        if deferred and launcher is not None:
            raise ValueError("the deferred mode drives the C ABI itself: no launcher can be injected")
        self.deferred = bool(deferred)
        self.share_weights = bool(share_weights)
        self.write_aggregate = bool(write_aggregate)
        self.batch_bytes = 0 if deferred else int(batch_bytes)
        if self.batch_bytes and launcher is not None:
            raise ValueError("batched launches drive the C ABI themselves: no launcher can be injected")
        self._batch_bytes_asked = self.batch_bytes
        self._bucket_bytes = {}                # batched mode: bucket index -> bytes of one VSW's buffer
        self._ready_bytes = 0
        self._groups_fired = 0
        self._plans = {}                       # batched mode: group of buckets -> its plan
        self._stream_cache = {}
        self.stats_level = sync.stats_level(stats_level) or L.STATS_SIMILARITY
        if self.stats_level == L.STATS_GRAM and len(batches) > L.STATS_GRAM_MAX_K:
            raise ValueError(f"statistics level 'gram' serves up to {L.STATS_GRAM_MAX_K} VSWs, not {len(batches)}: "
                             f"use 'full' and sync.gram() over the gradient buffers")
        self._ready = {}                       # deferred / batched mode: bucket index -> complete _Slot not launched yet
        self._vsw_streams = {}                 # VSW index -> the stream its hooks ran on in this step
        self._plan = None                      # the planned launch used last (deferred / batched mode)
        self.batches = tuple(batches)
        self.K = len(self.batches)
        self.opt = opt
        self.optimizer = None
        self.param_buckets = dict(param_buckets or {})   # bucket index -> dict(param=, state1=, state2=, bounds=, fanout=, agg_out=)
        self.step_count = 0
        self.lr_scale = 1.0
        self.accumulations = 1                 # micro-batches each VSW summed into its buckets (no_sync() steps + 1)
        self.grad_clip = float("inf")          # per-bucket norm bound (ShardGNMTAdam's grad_clip)
        self._launcher = launcher or self._launch_fused
        self._lock = threading.RLock()
        self._slots = {}
        self._main_stream = None
        self._n_launch_streams = max(1, int(launch_streams))
        self._sync_streams = []                # the launch streams; empty: VSW 0's own stream carries the launches
        self._sync_stream = stream
        self.launch_on_last_vsw = bool(launch_on_last_vsw)
        if self.launch_on_last_vsw and stream is not None:
            raise ValueError("launch_on_last_vsw puts the launches on the VSWs' own streams: no stream= beside it")
        self._bucket_stream = {}               # launch_on_last_vsw: bucket index -> stream of the VSW that completed it
        self.auto_finish = bool(auto_finish)
        self.interleave_moments = bool(interleave_moments)
        self._moment_home = {}                 # id(parameter) -> (MomentArena, first element, parameter): interleaved moments
        self._step_open = False                # something was handed over since the last end of step
        self._finishing = False                # an implied end of step is running
        self._last_done = []                   # one event per launch stream behind the launches of the step finished last
        self._replica_of = {}                  # id(parameter) -> VSW index (register_replicas)
        self._stream_vsw = {}                  # raw stream -> VSW index (replicas found by the stream their hooks run on)
        self._native_seen = {}                 # bucket index -> {k: what VSW k handed over natively in this step}
        self._calls = {}                       # bucket index -> prepared sync.BucketCall(s)
        self._args_cache = {}
        self._launch_streams = set()           # streams that carry launches of the current step
        self._errors = []
        self._momentum_ready = False           # SGD: the momentum buffers hold a first step
        self._bound_steps = {}                 # id -> optimizer.state dictionary whose 'step' follows step_count
        self.launched = 0                      # fused launches queued so far
        self.launched_with_opt = 0             # of them, launches that updated weights
        # Native meeting point (jabas_rdv_*): buckets that come with the same buffers step after step are
        # described to it after their first launch here; from then on a hook's hand-over is one foreign call.
        self._own_launcher = launcher is None
        self._rdv = None
        self._native = {}                      # bucket index -> (buffer addresses per VSW, elements, prepared call, dtype,
                                               #                  ids of VSW 0's parameters in the bucket or None)
        self._native_on_done = {}
        self._native_args = {}
        self._main_ptr = None
        self.native_launches = 0               # launches queued by the native meeting point
        if optimizer is not None:
            self.bind_optimizer(optimizer)

    # ------------------------------------------------------------------ launch streams
    @property
    def _sync_stream(self):
        return self._sync_streams[0] if self._sync_streams else None

    @_sync_stream.setter
    def _sync_stream(self, stream):
        if stream is None:
            self._sync_streams = []
            return
        extra = [torch.cuda.Stream(stream.device) for _ in range(self._n_launch_streams - 1)]
        self._sync_streams = [stream] + extra

    def _launch_stream(self, bucket_index=0):
        if self._sync_streams:
            return self._sync_streams[bucket_index % len(self._sync_streams)]
        if self.launch_on_last_vsw:
            own = self._bucket_stream.get(bucket_index)
            if own is not None:
                return own
        return self._main_stream

    # ------------------------------------------------------------------ who hands over what
    def install(self, device=None):
        """Makes this object the meeting point of ``device`` (default: the current GPU; "cpu" for host
        tensors) for hooks registered without a state of ours: ``dummy_hook`` with ``state=None`` and a main
        state nobody attached (the reference's own registration, jabas/train/trainer.py:452-468)."""
        with _installed_lock:
            _installed[_device_key("cuda" if device is None and torch.cuda.is_available() else device)] = weakref.ref(self)
        return self

    def uninstall(self):
        with _installed_lock:
            for key in [k for k, ref in _installed.items() if ref() is self or ref() is None]:
                del _installed[key]

    def register_replicas(self, models):
        """models[k]: VSW k's module (or DistributedDataParallel wrapper), in VSW order: a hook that is
        handed a bucket without a state finds the VSW index from the bucket's parameters. This is what makes
        the assignment deterministic; without it replicas are numbered in the order their streams first show
        up, which needs one stream per VSW and equal local batches."""
        models = list(models)
        if len(models) != self.K:
            raise ValueError(f"{self.K} VSWs, {len(models)} models")
        table = {}
        for k, m in enumerate(models):
            for p in m.parameters():
                if table.setdefault(id(p), k) != k:
                    raise ValueError("a parameter object belongs to two replicas")
        with self._lock:
            self._replica_of = table
            self._stream_vsw = {}
        return self

    def vsw_of(self, bucket, tensor):
        """VSW index of the replica a peer hook (``dummy_hook`` without a state) was called for."""
        params = getattr(bucket, "parameters", None)
        if self._replica_of and callable(params):
            try:
                return self._replica_of[id(params()[0])]
            except (KeyError, IndexError):
                raise RuntimeError("a bucket of a replica that register_replicas was not told about") from None
        raw = torch._C._cuda_getCurrentStream(tensor.get_device()) if tensor.is_cuda else ("host", threading.get_ident())
        with self._lock:
            k = self._stream_vsw.get(raw)
            if k is None:
                if len(set(self.batches)) > 1:
                    raise RuntimeError("VSWs with unequal local batches must be told apart: call register_replicas(models) "
                                       "or register the peers with VSWPeerState(local, k)")
                taken = set(self._stream_vsw.values())
                free = [j for j in range(1, self.K) if j not in taken]
                if not free:
                    raise RuntimeError(f"more peer replicas than the {self.K - 1} this meeting point expects, or two "
                                       "replicas on one stream: call register_replicas(models)")
                k = self._stream_vsw[raw] = free[0]
        return k

    # ------------------------------------------------------------------ optimizer binding
    def bind_optimizer(self, optimizer):
        """The optimizer object whose update the fused launches perform (overlap weight-sync mode).
        Hyperparameters are read from its ``param_groups`` at every step, so learning-rate policies and
        torch schedulers act on it as usual; its state dictionaries hold views of the state arenas; its
        own ``step`` is not called. A ``grad_clip`` attribute (ShardGNMTAdam,
        examples/gnmt/seq2seq/train/shard_optimizer.py:8-29) bounds every bucket's gradient norm."""
        from .train.trainer import opt_from_torch_optimizer
        if self.optimizer is optimizer:
            return self
        if self.optimizer is not None:
            raise RuntimeError("another optimizer is already bound")
        self.opt = opt_from_torch_optimizer(optimizer)
        self.optimizer = optimizer
        self._group_of = {id(p): gi for gi, g in enumerate(optimizer.param_groups) for p in g["params"]}
        self.grad_clip = float(getattr(optimizer, "grad_clip", float("inf")))
        if hasattr(optimizer, "register_load_state_dict_post_hook"):
            me = weakref.ref(self)

            def adopt(o):
                local = me()
                if local is not None and local.optimizer is o:
                    local._adopt_loaded_state()

            optimizer.register_load_state_dict_post_hook(adopt)
        return self

    def _adopt_loaded_state(self):
        """``optimizer.load_state_dict`` puts fresh tensors into ``optimizer.state``; the launches read the
        arenas. For every bucket already laid out the loaded moments are copied into its arenas (a parameter
        the checkpoint holds no state for starts from zeros, as it would in torch) and the optimizer's
        dictionaries show the arenas again; the step count follows the checkpoint's. Buckets laid out later
        take the loaded tensors over when they are bound."""
        bound = [pb for pb in self.param_buckets.values() if pb.get("params") is not None]
        if not bound:
            return
        device = bound[0]["param"].device
        torch.cuda.synchronize(device)
        sgd = self.opt["kind"] == "sgd"
        names = ("momentum_buffer",) if sgd else self._MOMENT_NAMES
        steps, loaded_momentum = set(), False
        self._bound_steps = {}
        with torch.no_grad():
            for pb in bound:
                for prm in pb["params"]:
                    st = self.optimizer.state[prm]
                    n = prm.numel()
                    home = self._moment_home.get(id(prm))
                    if home is not None:
                        arena, start, _ = home
                        for j, name in enumerate(names[:arena.ways]):
                            loaded = st.pop(name, None)
                            flat = (loaded.to(device=device, dtype=torch.float32).reshape(-1) if torch.is_tensor(loaded)
                                    else torch.zeros(n, dtype=torch.float32, device=device))
                            arena.write(j, flat, start)
                    else:
                        o = (prm.data_ptr() - pb["param"].data_ptr()) // 4
                        for name, key in zip(names, ("state1", "state2", "state3")):
                            if key not in pb:
                                continue
                            view = pb[key][o:o + n].view(prm.shape)
                            loaded = st.get(name)
                            if torch.is_tensor(loaded):
                                view.copy_(loaded)
                                loaded_momentum = loaded_momentum or name == "momentum_buffer"
                            else:
                                view.zero_()
                            st[name] = view
                    if not sgd:
                        if "step" in st:
                            steps.add(int(float(st["step"])))
                        self._bound_steps[id(st)] = st
        if len(steps) > 1:
            raise ValueError(f"parameters at different step counts {sorted(steps)}: one fused launch cannot mirror that")
        if sgd:
            self._momentum_ready = loaded_momentum
        else:
            self.step_count = steps.pop() if steps else 0
            for st in self._bound_steps.values():
                st["step"] = self.step_count
        self._refresh_hyperparameters()
        self._args_cache.clear()
        self._native_args.clear()
        torch.cuda.synchronize(device)

    _MOMENT_NAMES = ("exp_avg", "exp_avg_sq", "max_exp_avg_sq")

    def _hook_moments_into_state_dict(self):
        """Interleaved moments: the optimizer object shows them when it is asked for its state. Before its
        ``state_dict()`` packs ``optimizer.state`` every parameter gets copies of its moments under torch's names;
        afterwards the result keeps them (in shallow copies of the per-parameter dictionaries: torch packs the
        dictionaries themselves) and the optimizer's own dictionaries lose them again."""
        opt = self.optimizer
        if getattr(opt, "_jabas_moment_hooks", None) is not None:
            opt._jabas_moment_hooks = weakref.ref(self)
            return
        opt._jabas_moment_hooks = weakref.ref(self)

        def before(o):
            me = o._jabas_moment_hooks()
            if me is None or me.optimizer is not o:
                return
            homes = list(me._moment_home.values())
            if homes:
                torch.cuda.synchronize(homes[0][0].device)
            for arena, start, prm in homes:
                st = o.state[prm]
                for j, name in enumerate(me._MOMENT_NAMES[:arena.ways]):
                    st[name] = arena.read(j, start, prm.numel()).view(prm.shape)

        def after(o, state_dict):
            me = o._jabas_moment_hooks()
            if me is None or me.optimizer is not o:
                return state_dict
            state_dict["state"] = {idx: dict(st) for idx, st in state_dict["state"].items()}
            for _arena, _start, prm in list(me._moment_home.values()):
                st = o.state[prm]
                for name in me._MOMENT_NAMES:
                    st.pop(name, None)
            return state_dict

        opt.register_state_dict_pre_hook(before)
        opt.register_state_dict_post_hook(after)

    def _refresh_hyperparameters(self):
        if self.optimizer is None:
            return
        from .train.trainer import refresh_opt_from_torch_optimizer
        refresh_opt_from_torch_optimizer(self.opt, self.optimizer)

    def _bind_bucket(self, bucket_index, slot):
        """Arenas for the weights and optimizer state of one bucket's parameters, laid out like the
        bucket (built on the first launch of the bucket and again when DDP hands over other buffers, as
        after its bucket rebuild). Module parameters, replica parameters and ``optimizer.state`` tensors
        become views into the arenas, so the rest of the program keeps reading and writing them as
        before. Runs on the thread that queues the launch, after every VSW has published the bucket:
        each replica is past every use of these parameters in its backward pass."""
        b0 = slot.buckets[0]
        pb = self.param_buckets.get(bucket_index)
        if self.optimizer is None or b0 is None or not hasattr(b0, "parameters"):
            return pb
        # the buffers and the parameters they carry, in order (a bucket packs them back to back): DDP's bucket
        # rebuild frees the old buffers first, so new buckets can sit at old addresses with other contents
        params = list(b0.parameters())
        key = tuple(t.data_ptr() for t in slot.tensors) + (slot.tensors[0].numel(),) + tuple(id(p) for p in params)
        if pb is not None and pb.get("_key") == key:
            return pb
        buf0 = slot.tensors[0]
        es = buf0.element_size()
        offs = [(g.data_ptr() - buf0.data_ptr()) // es for g in b0.gradients()]
        n = buf0.numel()
        for p, o in zip(params, offs):
            if p.dtype != torch.float32:
                raise TypeError("the fused update keeps fp32 weights")
            if not 0 <= o <= n - p.numel():
                raise RuntimeError(f"bucket {bucket_index}: a gradient view lies outside the bucket buffer")
            if id(p) not in self._group_of:
                raise ValueError(f"bucket {bucket_index} carries a parameter no group of the optimizer holds")
        order = sorted(range(len(params)), key=lambda i: offs[i])
        sgd = self.opt["kind"] == "sgd"
        interleaved = self.interleave_moments and not sgd
        with torch.no_grad(), torch.cuda.stream(self._launch_stream(bucket_index)):
            new = dict(_key=key, param=_arena_like(buf0), fanout=[])
            if interleaved:
                # the bucket's first element at the element of a 256-byte line its other buffers start at
                first = (buf0.data_ptr() // es) % 64
                arena = sync.MomentArena(first + n, 3 if self.opt.get("amsgrad", False) else 2, buf0.device)
                new["moments"] = (arena, first)
            else:
                if not sgd or self.opt.get("momentum", 0.0) != 0.0:
                    new["state1"] = _arena_like(buf0)
                if not sgd:
                    new["state2"] = _arena_like(buf0)
                if self.opt.get("amsgrad", False):
                    new["state3"] = _arena_like(buf0)
            if buf0.dtype != torch.float32 and (self.write_aggregate or self.grad_clip != float("inf")):
                new["agg_out"] = _arena_like(buf0)
            names = ("momentum_buffer",) if sgd else ("exp_avg", "exp_avg_sq", "max_exp_avg_sq")
            had_state = 0
            for p, o in zip(params, offs):
                view = new["param"][o:o + p.numel()].view(p.shape)
                view.copy_(p.data)
                p.data = view
                st = self.optimizer.state[p]
                if interleaved:
                    arena, first = new["moments"]
                    home = self._moment_home.get(id(p))
                    for j, name in enumerate(names[:arena.ways]):
                        if torch.is_tensor(st.get(name)):               # carried in by the optimizer object
                            arena.write(j, st[name].to(buf0.device), first + o)
                        elif home is not None:                          # kept by the bucket the parameter was in before
                            arena.write(j, home[0].read(j, home[1], p.numel()), first + o)
                        st.pop(name, None)
                    self._moment_home[id(p)] = (arena, first + o, p)
                for name, arena in zip(names, ("state1", "state2", "state3")):
                    if arena not in new:
                        continue
                    sview = new[arena][o:o + p.numel()].view(p.shape)
                    if torch.is_tensor(st.get(name)):
                        sview.copy_(st[name])
                        had_state += name in ("momentum_buffer", "exp_avg")
                    st[name] = sview
                if not sgd:
                    if "step" in st and int(float(st["step"])) != self.step_count:
                        if self.launched_with_opt:
                            raise RuntimeError("a parameter's Adam step count differs from the steps taken here")
                        self.step_count = int(float(st["step"]))        # state carried in from earlier steps
                    st["step"] = self.step_count
                    self._bound_steps[id(st)] = st
            if sgd and had_state:
                if had_state != len(params) and self.opt.get("dampening", 0.0) != 0.0:
                    raise RuntimeError("some parameters of a bucket hold a momentum buffer and some do not: "
                                       "with dampening the first step of the latter cannot share a launch")
                self._momentum_ready = True
            for k in range(1, self.K):
                bk = slot.buckets[k]
                if bk is None or not hasattr(bk, "parameters"):
                    continue                                   # that replica's weights are not ours to refresh
                bufk = slot.tensors[k]
                peers = list(bk.parameters())
                poffs = [(g.data_ptr() - bufk.data_ptr()) // es for g in bk.gradients()]
                if poffs != offs or [q.shape for q in peers] != [p.shape for p in params]:
                    raise RuntimeError(f"bucket {bucket_index}: VSW {k} lays its parameters out differently from VSW 0")
                if self.share_weights:
                    for q, o in zip(peers, offs):
                        q.data = new["param"][o:o + q.numel()].view(q.shape)
                    continue
                arena = _arena_like(buf0)
                new["fanout"].append(arena)
                for q, o in zip(peers, offs):
                    view = arena[o:o + q.numel()].view(q.shape)
                    view.copy_(q.data)
                    q.data = view
        bounds = []
        for i in order:
            gi = self._group_of[id(params[i])]
            if not bounds:
                bounds.append((0, gi))
            elif bounds[-1][1] != gi:
                bounds.append((offs[i], gi))
        new["bounds"] = tuple(bounds)
        new["params"] = params
        self.param_buckets[bucket_index] = new
        if interleaved:
            self._hook_moments_into_state_dict()
        with self._lock:
            self._calls.pop(bucket_index, None)
            self._plans.clear()
        self._forget_native(bucket_index)
        return new

    def aggregate_of(self, bucket_index):
        """The fp32 aggregate of a reduced-precision bucket (fp32 buckets hold theirs in place)."""
        pb = self.param_buckets.get(bucket_index) or {}
        return pb.get("agg_out")

    # ------------------------------------------------------------------ hooks call this
    def publish(self, k, bucket_index, tensor, want_stats=False, on_done=None, value=None, bucket=None, _stream=None):
        """Hands VSW k's bucket ``bucket_index`` over; the fused launch for that bucket is
        queued by whichever VSW hands its bucket over last. Returns a completed Future
        carrying ``value`` (default the tensor). ``bucket``: the bucket object itself, whose
        ``parameters()`` / ``gradients()`` place the weights when an optimizer is bound and whose
        ``is_last()`` ends the step (``auto_finish``). ``_stream``: the VSW's stream when the hand-over is
        repeated on its behalf by another thread (a bucket leaving the native meeting point)."""
        if not 0 <= k < self.K:
            raise ValueError(f"VSW index {k} outside 0..{self.K - 1}")
        if self._finishing:                    # an implied end of step is running on another thread: let it finish
            with self._lock:
                pass
        self._step_open = True
        fut = torch.futures.Future()
        fut.set_result(tensor if value is None else value)
        known = self._native.get(bucket_index)
        if known is not None and tensor.is_cuda and _stream is None:
            if known[0][k] == tensor.data_ptr() and known[1] == tensor.numel() and self._same_parameters(k, bucket, known):
                if self._publish_native(k, bucket_index, tensor, want_stats, on_done, known, bucket):
                    self._end_of_step(bucket)
                return fut
            self._leave_native(bucket_index, k)
        event = stream = None
        if tensor.is_cuda:
            stream = self._current_stream(tensor) if _stream is None else _stream
            if not self.deferred and not self.batch_bytes and (k != 0 or self._sync_stream is not None
                                                                or self.launch_on_last_vsw):
                # VSW 0's own stream needs none when the launch is queued on it. A fresh event every time:
                # recording one event again step after step (to save its creation) made the waits on it
                # three times as expensive on this runtime. (Batched and deferred launches order themselves
                # behind one event per VSW stream, recorded when the launch is queued.)
                event = torch.cuda.Event()
                event.record(stream)
        batch = None
        with self._lock:
            if stream is not None:
                self._vsw_streams[k] = stream  # deferred mode orders once per VSW stream in finish_step
            slot = self._slots.get(bucket_index)
            if slot is None:
                slot = self._slots[bucket_index] = _Slot(self.K)
            if slot.tensors[k] is not None:
                raise RuntimeError(f"VSW {k} published bucket {bucket_index} twice in one step")
            slot.tensors[k], slot.events[k], slot.buckets[k] = tensor, event, bucket
            slot.count += 1
            if k == 0:
                slot.want_stats, slot.on_done = want_stats, on_done
                self._main_stream = stream
                self._main_ptr = None if stream is None else stream.cuda_stream
            complete = ready = slot.count == self.K
            if ready:
                del self._slots[bucket_index]
                if self.launch_on_last_vsw and stream is not None and not self._sync_streams:
                    self._bucket_stream[bucket_index] = stream     # the launch follows this VSW's own work
                    slot.events[k] = None
                if self._batch_bytes_asked and stream is not None:
                    self._bucket_bytes[bucket_index] = tensor.numel() * tensor.element_size()
                if self.deferred or (self.batch_bytes and stream is not None):
                    self._ready[bucket_index] = slot
                    self._ready_bytes += tensor.numel() * tensor.element_size()
                    if not self.deferred and self._ready_bytes >= self.batch_bytes:
                        batch, self._ready, self._ready_bytes = self._ready, {}, 0
                    ready = False
        if ready:
            self._fire(bucket_index, slot)
        elif batch is not None:
            self._fire_group(batch)
        if complete:
            self._end_of_step(bucket)
        return fut

    def _end_of_step(self, bucket):
        """Called by the hand-over that completed a bucket: when that bucket is the replicas' last one, every
        launch of the step is queued (DDP hands a replica's buckets over in order), and the step ends here."""
        is_last = getattr(bucket, "is_last", None)
        if not self.auto_finish or not callable(is_last) or not is_last():
            return
        with self._lock:
            self._finishing = True
            try:
                self.finish_step()
            finally:
                self._finishing = False

    def _current_stream(self, tensor):
        """torch.cuda.current_stream(tensor.device) without its per-call device bookkeeping (4.6 us a call,
        as much as the rest of a publish): the Stream object of a raw stream is made once and kept."""
        return self._current_stream_and_ptr(tensor)[0]

    def _current_stream_and_ptr(self, tensor):
        raw = torch._C._cuda_getCurrentStream(tensor.get_device())
        hit = self._stream_cache.get(raw)
        if hit is None:
            stream = torch.cuda.Stream(stream_id=raw[0], device_index=raw[1], device_type=raw[2])
            hit = self._stream_cache[raw] = (stream, stream.cuda_stream)
        return hit

    # ------------------------------------------------------------------ native meeting point
    def _describe_native(self, bucket_index, tensors, call):
        """Describes a bucket that has just had its first launch from here to the native rendezvous."""
        dev = tensors[0].device
        lib = L.lib()
        with torch.cuda.device(dev), torch.cuda.stream(self._launch_stream(bucket_index)):
            if self._rdv is None:
                handle = C.c_void_p()
                L.check(lib.jabas_rdv_create(self.K, C.byref(handle)), "jabas_rdv_create")
                self._rdv = handle
                self._rdv_publish = lib.jabas_rdv_publish
            call.prepare_stats()
            L.check(lib.jabas_rdv_set_bucket(self._rdv, bucket_index, C.byref(call.c_span),
                                             None if call.bounds_dev is None else call.bounds_dev.data_ptr(),
                                             call._rows.data_ptr(), call.ws.buf.data_ptr(), call.ws.nbytes, call._flip),
                    "jabas_rdv_set_bucket")
        # With weights behind the bucket the description is only good for the parameters it was made for, in their
        # order: DDP's bucket rebuild can put other parameters at the old addresses, and the span's group bounds,
        # the arenas and the replicas' views would silently belong to the old ones.
        pb = self.param_buckets.get(bucket_index) or {}
        sig = tuple(id(p) for p in pb["params"]) if call.with_opt and pb.get("params") is not None else None
        self._native[bucket_index] = (tuple(t.data_ptr() for t in tensors), tensors[0].numel(), call, tensors[0].dtype, sig)

    @staticmethod
    def _same_parameters(k, bucket, known):
        """Whether VSW 0's bucket still carries the parameters the native description was made for (every
        replica rebuilds its buckets alike, so VSW 0's word covers the others)."""
        sig = known[4]
        if sig is None or k != 0:
            return True
        params = getattr(bucket, "parameters", None)
        return callable(params) and tuple(id(p) for p in params()) == sig

    def _leave_native(self, bucket_index, k):
        """A VSW came with another buffer (or other parameters) than the native description holds: the
        description is dropped and whoever has already handed the bucket over natively in this step is handed
        over again on the Python path, on its own stream (an event recorded now covers everything the earlier
        one covered)."""
        with self._lock:
            seen = self._native_seen.pop(bucket_index, {})
        arrived = self._forget_native(bucket_index)
        if arrived != len(seen):
            raise RuntimeError(f"bucket {bucket_index}: VSW {k} handed over another buffer than in the step before, "
                               f"after {arrived} other VSW(s) had handed over the same ones as before")
        for j, (tensor, bucket, want_stats, on_done, stream) in sorted(seen.items()):
            self.publish(j, bucket_index, tensor, want_stats=want_stats, on_done=on_done, bucket=bucket, _stream=stream)

    def _forget_native(self, bucket_index):
        """Drops the native description; returns how many VSWs had handed the bucket over natively in this step."""
        known = self._native.pop(bucket_index, None)
        if known is None or self._rdv is None:
            return 0
        return max(0, L.lib().jabas_rdv_drop_bucket(self._rdv, bucket_index))

    def _publish_native(self, k, bucket_index, tensor, want_stats, on_done, known, bucket=None):
        """One hand-over at the native meeting point; True when this call completed the bucket."""
        stream, ptr = self._current_stream_and_ptr(tensor)
        self._vsw_streams[k] = stream
        seen = self._native_seen.get(bucket_index)
        if seen is None:
            seen = self._native_seen.setdefault(bucket_index, {})
        seen[k] = (tensor, bucket, want_stats, on_done, stream)
        if k == 0:
            self._main_stream, self._main_ptr = stream, ptr
            self._native_on_done[bucket_index] = on_done
        if self._sync_streams:
            launch = self._launch_stream(bucket_index)
            main_ptr = launch.cuda_stream
        elif self.launch_on_last_vsw:
            launch, main_ptr = stream, ptr                      # used only if this hand-over completes the bucket
        else:
            launch, main_ptr = self._main_stream, self._main_ptr
        call = known[2]
        stamp = (self.step_count, self.lr_scale, self.accumulations)
        ent = self._native_args.get((known[3], call.with_opt))
        if ent is None or ent[0] != stamp:
            args = self._step_args(known[3], False, call.with_opt)
            ent = self._native_args[(known[3], call.with_opt)] = (stamp, args, C.byref(args))
        rc = self._rdv_publish(self._rdv, k, bucket_index, 1 if want_stats else 0, ptr, main_ptr, ent[2], self.stats_level)
        if rc == L.RDV_WAITING:
            return False
        if rc < 0 or rc == L.RDV_UNKNOWN:
            with self._lock:
                self._errors.append((bucket_index, L.JabasSyncError(rc if rc < 0 else L.ERR_STATE, "jabas_rdv_publish")))
            return False
        if rc >= L.RDV_LAUNCHED_ROW0:
            call._flip = rc - L.RDV_LAUNCHED_ROW0          # the Python path continues the alternation from here
        row = call._rows[rc - L.RDV_LAUNCHED_ROW0] if rc >= L.RDV_LAUNCHED_ROW0 else None
        with self._lock:
            self._native_seen.pop(bucket_index, None)
            if self.launch_on_last_vsw and not self._sync_streams:
                self._bucket_stream[bucket_index] = launch
            self._launch_streams.add(launch)
            self.launched += 1
            self.native_launches += 1
            if call.with_opt:
                self.launched_with_opt += 1
        done = self._native_on_done.get(bucket_index)
        if done is not None:
            done(BucketStats(bucket_index, row) if row is not None else None)
        return True

    def _fire(self, bucket_index, slot):
        main = self._launch_stream(bucket_index)
        try:
            if main is not None:
                for ev in slot.events:
                    if ev is not None:
                        main.wait_event(ev)
                self._bind_bucket(bucket_index, slot)
                row = self._launcher(bucket_index, slot.tensors, slot.want_stats)
                with self._lock:
                    self._launch_streams.add(main)
            else:
                row = self._launcher(bucket_index, slot.tensors, slot.want_stats)
        except Exception as exc:                       # reported by finish_step
            with self._lock:
                self._errors.append((bucket_index, exc))
            return
        if slot.on_done is not None:
            slot.on_done(BucketStats(bucket_index, row) if row is not None else None)
        with self._lock:
            self.launched += 1

    # ------------------------------------------------------------- the default launcher
    def _step_args(self, dtype, want_stats, with_opt, grad_scale=None, batches=None):
        """JabasStepArgs of this step, built once per (step, kind of launch) and shared by its buckets."""
        key = (self.step_count, self.lr_scale, self.accumulations, dtype, bool(want_stats), bool(with_opt),
               None if grad_scale is None else grad_scale.data_ptr(), batches)
        with self._lock:
            hit = self._args_cache.get(key)
            if hit is None:
                if len(self._args_cache) > 64:
                    self._args_cache.clear()
                if with_opt and not self._args_cache_fresh:
                    self._refresh_hyperparameters()
                    self._args_cache_fresh = True
                hit = self._args_cache[key] = sync.make_step_args(
                    self.batches if batches is None else batches, dtype, stats=self.stats_level if want_stats else 0,
                    opt=self.opt if with_opt else None, step=self.step_count + 1,
                    first_step=not self._momentum_ready, lr_scale=self.lr_scale,
                    accumulations=self.accumulations if batches is None else 1, grad_scale=grad_scale)
        return hit

    _args_cache_fresh = False

    def _launch_fused(self, bucket_index, tensors, want_stats):
        """Queues ``jabas_sync_bucket`` for one bucket on the launch stream. DDP hands a hook the same
        bucket buffers every step, so the prepared call (validated span, C struct, device bound table,
        workspace) is kept per bucket and rebuilt only when the buffers change.

        With a finite ``grad_clip`` (the per-bucket clipping of ShardGNMTAdam.step,
        examples/gnmt/seq2seq/train/shard_optimizer.py:75-76) the bucket takes two launches: aggregate +
        statistics, the coefficient max_norm / (norm + 1e-6) on the device, then the update over the
        aggregate scaled by it: the norm has to be known before any weight moves."""
        main = self._launch_stream(bucket_index)
        with self._lock:
            call = self._calls.get(bucket_index)
        if call is None or not call.matches(tensors):
            span, with_opt = self._span_of(bucket_index, tensors)
            clipped = with_opt and self.grad_clip != float("inf")
            if clipped:
                agg_span = sync.SpanSpec(tensors, agg_out=span.agg_out)
                call = sync.BucketCall(agg_span)
                call.update = sync.BucketCall(sync.SpanSpec(
                    [span.agg_out], agg_out=span.agg_out, param=span.param, state1=span.state1, state2=span.state2,
                    state3=span.state3, fanout=span.fanout, bounds=span.bounds, moments=span.moments))
                with torch.cuda.stream(main):
                    call.coef = torch.ones(1, dtype=torch.float32, device=tensors[0].device)
            else:
                call = sync.BucketCall(span)
            call.with_opt, call.clipped = with_opt, clipped
            with self._lock:
                self._calls[bucket_index] = call
            describe = self._own_launcher and not self.deferred and not self.batch_bytes and not clipped and main is not None
        else:
            describe = False
        if call.with_opt:
            with self._lock:
                self.launched_with_opt += 1
        if not call.clipped:
            row = call.run(self._step_args(tensors[0].dtype, want_stats, call.with_opt), stream=main)
            if describe:                                # after the launch: the description continues from the row it wrote
                self._describe_native(bucket_index, tensors, call)
            return row
        row = call.run(self._step_args(tensors[0].dtype, True, False), stream=main)
        sync.clip_coef(row, self.grad_clip, out=call.coef, stream=main)
        call.update.run(self._step_args(torch.float32, False, True, grad_scale=call.coef, batches=(1,)), stream=main)
        return row if want_stats else None

    def _span_of(self, bucket_index, tensors):
        """(span over the K buffers of one bucket, whether the optimizer runs in the same launch)."""
        g0 = tensors[0]
        pb = self.param_buckets.get(bucket_index)
        opt = self.opt if pb is not None else None
        agg_out = g0 if g0.dtype == torch.float32 else (pb or {}).get("agg_out")
        if opt is not None and self.grad_clip != float("inf") and agg_out is None:
            raise ValueError("clipping a reduced-precision bucket needs an fp32 agg_out arena")
        if opt is not None and not self.write_aggregate and self.grad_clip == float("inf"):
            agg_out = None
        span = sync.SpanSpec(tensors, agg_out=agg_out,
                             param=pb and pb.get("param"), state1=pb and pb.get("state1"),
                             state2=pb and pb.get("state2"), state3=pb and pb.get("state3"),
                             moments=pb and pb.get("moments"),
                             fanout=(pb or {}).get("fanout", ()),
                             bounds=(pb or {}).get("bounds", ()) if opt else ())
        return span, opt is not None

    def _fire_group(self, ready):
        """One planned launch over a group of complete buckets, in bucket order: all buckets of the step
        (deferred mode, from ``finish_step``) or a batch of them (batched mode). The launch is ordered behind
        one event per VSW stream, recorded here: every VSW has handed over all buckets of the group, so
        whatever its stream holds by now includes the work that filled them (and at most the few kernels its
        thread has queued since). A fresh event per hand-over, of which only each VSW's last would be waited
        for, cost the hooks 5 us each: 1.5 ms of host time per ViT-L/16 step."""
        with self._lock:
            vsw_streams = sorted(self._vsw_streams.items())
        order = sorted(ready)
        slots = [ready[i] for i in order]
        main = self._launch_stream(0 if self.deferred else self._groups_fired)
        self._groups_fired += 1
        if main is None:
            for i, slot in zip(order, slots):          # host tensors (protocol tests)
                self._fire(i, slot)
            return
        try:
            # one event per stream instead of one per bucket and VSW, which on the GPU's queue are a barrier
            # packet each (98 of them per step for 14 buckets x 4 VSWs cost 0.25 ms)
            for k, stream in vsw_streams:
                if stream != main:
                    ev = torch.cuda.Event()
                    ev.record(stream)
                    main.wait_event(ev)
            for i, slot in zip(order, slots):
                self._bind_bucket(i, slot)
        except Exception as exc:
            with self._lock:
                self._errors.append((order[0], exc))
            return
        with_opt = [self.opt is not None and i in self.param_buckets for i in order]
        if (any(with_opt) and not all(with_opt)) or (with_opt[0] and self.grad_clip != float("inf")):
            gate, gated = None, {main}
            for i, slot in zip(order, slots):          # buckets with and without weights behind them, or a norm
                slot.events = [None] * self.K          # per bucket to wait for: one launch each after all
                own = self._launch_stream(i)           # the VSW streams were ordered ahead of `main` only
                if own not in gated:
                    if gate is None:
                        gate = torch.cuda.Event()
                        gate.record(main)
                    own.wait_event(gate)
                    gated.add(own)
                self._fire(i, slot)
            return
        try:
            key = tuple((i, slot.tensors[0].numel()) + tuple(t.data_ptr() for t in slot.tensors)
                        for i, slot in zip(order, slots))
            with self._lock:
                plan = self._plans.get(key)
            if plan is None:                            # DDP hands over the same buffers every step: built once
                spans = [self._span_of(i, slot.tensors)[0] for i, slot in zip(order, slots)]
                plan = sync.SyncPlan(spans, sync.opt_kind(self.opt) if with_opt[0] else L.OPT_NONE)
                with self._lock:
                    if len(self._plans) >= 256:
                        self._plans.clear()
                    self._plans[key] = plan
            self._plan = plan
            want = any(slot.want_stats for slot in slots)
            args = self._step_args(slots[0].tensors[0].dtype, want, with_opt[0])
            rows = plan.run(args, stream=main)
            if rows is not None:
                with torch.cuda.stream(main):
                    rows = rows.clone()                 # the plan's own rows are overwritten by its next launch
            with self._lock:
                if with_opt[0]:
                    self.launched_with_opt += 1
                self._launch_streams.add(main)
        except Exception as exc:
            with self._lock:
                self._errors.append((order[0], exc))
            return
        for j, (i, slot) in enumerate(zip(order, slots)):
            if slot.on_done is not None:
                slot.on_done(BucketStats(i, rows[j]) if slot.want_stats and rows is not None else None)
        with self._lock:
            self.launched += 1

    # ------------------------------------------------------------------ trainer calls this
    def pending(self):
        with self._lock:
            return sorted(self._slots)

    def reset(self):
        """Forgets the buckets of an unfinished step (after an error), so that the next step starts clean."""
        with self._lock:
            self._slots.clear()
            self._ready.clear()
            self._ready_bytes = 0
            self._launch_streams = set()
            self._vsw_streams = {}
            self._errors = []
            self._step_open = False
        self._reset_native()

    def _reset_native(self):
        """Clears the native meeting point; returns how many of its buckets were incomplete."""
        self._native_seen = {}
        return 0 if self._rdv is None else max(0, L.lib().jabas_rdv_reset(self._rdv))

    def __del__(self):
        rdv, self._rdv = getattr(self, "_rdv", None), None
        if rdv is not None:
            try:
                L.lib().jabas_rdv_destroy(rdv)
            except Exception:                          # interpreter shutdown
                pass

    def finish_step(self, streams=()):
        """End of a sync step: every VSW stream waits for the fused launches that read its
        buckets (and, with an optimizer bound, write its weights), and the step count (Adam's t, SGD's
        first-step flag) advances. ``streams``: the VSW streams; default: the streams the hooks of this
        step ran on. A step that the last bucket's hand-over has already ended (``auto_finish``) is not ended
        twice: the call only orders ``streams`` behind that step's launches."""
        if not self._step_open:
            for done in self._last_done:
                for s in streams:
                    s.wait_event(done)
            return
        self._step_open = False
        left = self.pending()
        left_native = self._reset_native()
        if left or left_native:
            self.reset()
            raise RuntimeError(f"buckets {left} were not published by every VSW" +
                               (f" ({left_native} more at the native meeting point)" if left_native else ""))
        with self._lock:
            ready, self._ready, self._ready_bytes = self._ready, {}, 0
        if ready:
            self._fire_group(ready)
        # the launches of a step sit on one stream in order: one event behind the last of them orders
        # every VSW stream behind all of them
        with self._lock:
            launch_streams, self._launch_streams = self._launch_streams, set()
            recorded, self._vsw_streams = self._vsw_streams, {}
            errors, self._errors = self._errors, []
            self._args_cache_fresh = False
        streams = tuple(streams) or tuple(recorded.values())
        self._last_done = []
        for main in launch_streams:
            done = torch.cuda.Event()
            done.record(main)
            self._last_done.append(done)
            for s in streams:
                if s != main:
                    s.wait_event(done)
        if self._batch_bytes_asked and self.batch_bytes and self._bucket_bytes:
            # Batching pays by merging several short launches into one; when a batch would hold fewer than two
            # buckets on average it merges nothing and only holds buckets back (measured on the GNMT set, 11
            # buckets of 58 MB on average in 64 MiB batches: 1.55 ms a step against 1.52 one launch per bucket).
            mean = sum(self._bucket_bytes.values()) / len(self._bucket_bytes)
            if 2 * mean > self._batch_bytes_asked:
                self.batch_bytes = 0
        if errors:
            idx, exc = errors[0]
            self.reset()
            raise RuntimeError(f"fused launch of bucket {idx} failed: {exc}") from exc
        self.step_count += 1
        if self.launched_with_opt:
            self._momentum_ready = True
        for st in self._bound_steps.values():
            st["step"] = self.step_count
