"""The part of the IIDP/JABAS trainer that sits on the gradient-sync path, for one GPU.

``VSWSyncTrainer`` mirrors the attributes and call order through which the reference
reaches the path (jabas/train/trainer.py: ``prepare_stream_parallel`` :82-86,
``prepare_weight_sync_method`` :88-98, ``compute`` :171-174, ``step`` :176-197,
``_compute_cosine_similarity`` :470-483, ``_adjust_adaptive_lr`` :693-700; attributes
``local_models``, ``main_model``, ``local_optimizers``, ``main_optimizer``, ``local_schedulers``,
``model_streams``, ``num_models``, ``sync_step``, ``similarity_state``, ``cos_placeholder``):
K model replicas on K HIP streams, one sync step per iteration. The optimizer object the
caller hands to ``prepare_weight_sync_method`` stays the place where hyperparameters live
(``main_optimizer.param_groups[i]['lr']`` is read at every step, so the reference's learning-rate
policies and torch LR schedulers work unchanged) and where the state is visible
(``main_optimizer.state[p]`` holds views of the state arenas, so ``state_dict()`` checkpoints it);
its own ``step()`` is never called: the fused launch does the update.
It is not the reference's trainer: data loading, the configuration solver, elastic
restarts and the cross-GPU all-reduce are outside this build.

Memory layout (MI355X-first): the weights, their optimizer state and every VSW's gradient
buckets live in flat arenas with one common bucket layout (``VSWFlatSync``). The parameters
of every VSW's model are views of ONE weight arena (no copy of the new weights to the other
VSWs), a VSW's gradients are moved into its buckets by one multi-tensor launch per backward
pass (no clearing of the buckets between steps), and the whole sync step is one fused launch
that writes nothing but the weights and the optimizer state.
"""
import copy
import weakref

import torch

from ..engine import VSWFlatSync
from ..workloads import ParamSpec
from ..ddp_comm_hooks import GradientSimilarityState
from .. import sync


def create_optimizer_hook(hook, optimizer):
    """Counterpart of IIDPTrainer._create_optimizer_hook (call site jabas/train/trainer.py:332): the
    hook VSW 0 registers in the overlap weight-sync mode, which updates the parameters of a bucket as
    soon as the bucket's gradients are synchronised.

    With a ``LocalBucketSync`` attached to the state (K VSWs on the GPU) the optimizer is bound to it and
    the update is part of the fused launch the rendezvous queues for that bucket, when the last VSW has
    handed its bucket over, on the rendezvous' launch stream: aggregate, ``optimizer``'s update rule and
    the refresh of the other replicas' weights in one pass. ``optimizer.step`` itself is never called;
    its ``param_groups`` supply the hyperparameters at every step and its ``state`` shows the arenas.
    Calling ``optimizer.step`` on this thread right after ``hook`` would read VSW 0's own bucket before
    the other VSWs' gradients are in it.

    Without a rendezvous (state None or a one-worker state) the bucket already holds the final gradient
    when the hook's Future resolves, and ``optimizer.step(gradients)`` runs then, gradients tagged with
    the ``.index`` of their parameters the way the reference matches them
    (examples/gnmt/seq2seq/train/shard_optimizer.py:41-46)."""
    def hook_then_step(state, bucket):
        local = getattr(state, "local", None)
        if local is None:                  # a state built as the reference builds it: the device's meeting point
            from ..ddp_comm_hooks.default_hooks import bucket_tensor, installed_local
            local = installed_local(bucket_tensor(bucket))
            if local is not None and state is not None:
                state.local = local
        if local is not None:
            local.bind_optimizer(optimizer)
            return hook(state, bucket)
        if getattr(state, "total_num_decoupled_workers", 1) != 1:
            raise RuntimeError("create_optimizer_hook: several workers but no LocalBucketSync attached to the state")
        fut = hook(state, bucket)

        def run(done):
            value = done.value()
            params, grads = bucket.parameters(), bucket.gradients()
            for p, g in zip(params, grads):
                if not isinstance(getattr(p, "index", None), int):
                    raise RuntimeError("parameters need an .index attribute (see tag_parameter_indices)")
                g.index = p.index
            optimizer.step(grads)
            return value

        return fut.then(run)
    return hook_then_step


def create_stream_for_optimizer(device=None):
    """Counterpart of IIDPTrainer._create_stream_for_optimizer (call site jabas/train/trainer.py:328): the
    stream the weight updates of the overlap mode run on, apart from every VSW's own stream, so that a
    bucket's update overlaps the rest of the backward passes. Default priority."""
    return torch.cuda.Stream(device)


def prepare_overlap_optimizer_with_ddp(local_models, states, hooks, optimizer, local):
    """jabas/train/trainer.py:327-333 for one GPU: launch streams of its own for ``local`` (the GPU's
    LocalBucketSync) unless it has them, ``local`` installed as the device's meeting point with the replicas
    registered in VSW order, the optimizer hook on VSW 0, every other VSW's hook as it is.
    ``local_models`` are the K DistributedDataParallel replicas (built with
    ``gradient_as_bucket_view=True``: the fused launch writes the aggregate into the bucket, and only a
    ``.grad`` that is a view of the bucket sees it)."""
    p = next(iter(local_models[0].parameters()))
    if local._sync_stream is None:
        local._sync_stream = create_stream_for_optimizer(p.device)
    # states built without a handle of ours (the reference's: a plain GradientSimilarityState and None for every
    # other VSW, jabas/train/trainer.py:452-468) find the meeting point through the device and the VSW index
    # through the replica a bucket's parameters belong to
    local.install(p.device)
    local.register_replicas(local_models)
    for i, (model, state, hook) in enumerate(zip(local_models, states, hooks)):
        if getattr(model, "gradient_as_bucket_view", True) is False:
            raise ValueError("build the DistributedDataParallel replicas with gradient_as_bucket_view=True")
        if i == 0:
            local.bind_optimizer(optimizer)
            hook = create_optimizer_hook(hook, optimizer)
        model.register_comm_hook(state=state, hook=hook)
    return local


def tag_parameter_indices(model):
    """Gives every parameter the ``.index`` the Shard optimizers match on."""
    for i, p in enumerate(model.parameters()):
        p.index = i
    return model


def opt_from_torch_optimizer(optimizer):
    """Hyperparameter dictionary (the form ``sync.make_step_args`` takes) of a torch.optim.SGD / Adam /
    AdamW or a jabas_amd.optim.Shard* object. One momentum / betas / eps for all groups, as the
    kernel takes them per launch; learning rate and weight decay per group."""
    from ..optim import ShardSGD, ShardAdam, ShardAdamW
    groups = optimizer.param_groups
    if not groups:
        raise ValueError("optimizer has no parameter groups")
    g0 = groups[0]

    def same(key):
        vals = [g[key] for g in groups]
        if any(v != vals[0] for v in vals[1:]):
            raise ValueError(f"parameter groups differ in {key!r}: one value per launch is supported")
        return vals[0]

    if isinstance(optimizer, (torch.optim.SGD, ShardSGD)):
        opt = dict(kind="sgd", momentum=float(same("momentum")), dampening=float(same("dampening")),
                   nesterov=bool(same("nesterov")))
        if g0.get("maximize", False):
            raise ValueError("maximize=True is not supported")
    elif isinstance(optimizer, (torch.optim.AdamW, ShardAdamW, torch.optim.Adam, ShardAdam)):
        adamw = isinstance(optimizer, (torch.optim.AdamW, ShardAdamW))
        if g0.get("maximize", False):
            raise ValueError("maximize=True is not supported")
        b1, b2 = same("betas")
        opt = dict(kind="adamw" if adamw else "adam", betas=(float(b1), float(b2)), eps=float(same("eps")),
                   amsgrad=bool(same("amsgrad")) if "amsgrad" in g0 else False)
    else:
        raise TypeError(f"unsupported optimizer type {type(optimizer).__name__}: SGD, Adam, AdamW or their "
                        "Shard counterparts")
    opt["groups"] = [dict(lr=float(g["lr"]), weight_decay=float(g.get("weight_decay", 0.0))) for g in groups]
    return opt


def refresh_opt_from_torch_optimizer(opt, optimizer):
    """Brings the hyperparameter dictionary ``opt`` (made by ``opt_from_torch_optimizer``) up to what the optimizer
    object's ``param_groups`` hold now: learning rate and weight decay per group, and the values a launch takes
    once (momentum / dampening / nesterov, betas / eps), which schedulers that cycle the momentum move from step
    to step. Groups that have come to differ in one of the latter, and a momentum that appears or disappears (the
    momentum buffer exists or it does not), are errors."""
    groups = optimizer.param_groups
    for mine, theirs in zip(opt["groups"], groups):
        mine["lr"] = float(theirs["lr"])
        mine["weight_decay"] = float(theirs.get("weight_decay", 0.0))
    g0 = groups[0]
    keys = ("momentum", "dampening", "nesterov") if opt["kind"] == "sgd" else ("betas", "eps")
    for key in keys:
        if key not in g0:
            continue
        for g in groups[1:]:
            if g[key] != g0[key]:
                raise ValueError(f"parameter groups differ in {key!r}: one value per launch is supported")
    if opt["kind"] == "sgd":
        momentum = float(g0.get("momentum", opt.get("momentum", 0.0)))
        if (momentum != 0.0) != (opt.get("momentum", 0.0) != 0.0):
            raise ValueError("the momentum became zero or non-zero after the state arenas were laid out")
        opt["momentum"] = momentum
        opt["dampening"] = float(g0.get("dampening", opt.get("dampening", 0.0)))
        opt["nesterov"] = bool(g0.get("nesterov", opt.get("nesterov", False)))
    else:
        if "betas" in g0:
            opt["betas"] = (float(g0["betas"][0]), float(g0["betas"][1]))
        if "eps" in g0:
            opt["eps"] = float(g0["eps"])


class VSWSyncTrainer:
    def __init__(self, gpu, local_batch_sizes, opt=None, interval=100, grad_dtype=torch.float32,
                 param_groups_func=None, similarity_target=None, controller=None, clip_norm=None,
                 share_weights=True, keep_grads=False, interleave_moments=True):
        """opt: hyperparameter dictionary, or None when an optimizer object follows through
        ``prepare_weight_sync_method`` (the reference's order of calls).

        share_weights: the parameters of every VSW's model are views of ONE weight arena. The VSWs of a GPU
        hold identical weights after every step (IIDP copies the main VSW's weights to the others), and no
        VSW reads weights while the step runs (the launch waits for all K backward passes), so one copy serves
        them all: nothing is written per replica (4 (K - 1) bytes per element and step saved: 28 of 72 for
        eight VSWs) and K - 1 copies of the model's weights stay out of HBM. False: one weight arena per
        VSW, refreshed by the launch (the reference's layout: separate modules with separate storage).

        keep_grads: after ``step()`` the ``.grad`` of the main model's parameters shows the synchronised gradient
        (views of the aggregate arena, the clipped values under a norm bound), as the reference leaves the averaged
        gradient in the main VSW's ``.grad`` for code that logs gradient norms or inspects gradients after the step;
        the launch then writes the aggregate (4 more bytes per element). Default: ``.grad`` is None after a step and
        the aggregate is written nowhere.

        interleave_moments: Adam's moments live in one arena of alternating blocks (``sync.MomentArena``), which the
        kernels stream 2-6 % faster than arrays of their own. The moments then are no flat tensors: the caller's
        optimizer object gets copies of them under torch's names whenever its ``state_dict()`` is called (and
        ``load_state_dict`` scatters them back), but ``optimizer.state[p]`` holds only the step count in between.
        False: flat state arenas, ``optimizer.state[p]["exp_avg"]`` etc. are live views at all times."""
        self.share_weights = bool(share_weights)
        self.keep_grads = bool(keep_grads)
        self.interleave_moments = bool(interleave_moments)
        self.gpu = torch.device("cuda", gpu) if isinstance(gpu, int) else torch.device(gpu)
        self.local_batch_sizes = tuple(local_batch_sizes)
        self.num_models = len(self.local_batch_sizes)
        self.total_num_decoupled_workers = self.num_models
        self.opt = opt
        self.grad_dtype = grad_dtype
        self.param_groups_func = param_groups_func
        self.similarity_target = similarity_target
        self.controller = controller              # AdaptiveBatchController or None (enable_adjust off)
        self.clip_norm = clip_norm
        self.global_lr_modifier = 1.0
        self.local_models, self.model_streams = [], []
        self.local_optimizers, self.local_schedulers = [], []
        self.main_model = self.main_optimizer = None
        self.sync_step = 0
        self.accumulated = 0                      # compute() calls since the last step (IIDP's accum_step + 1 at step time)
        self.engine = None
        self._bucket_views = {}                   # VSW index -> its bucket views, one per parameter
        self._params = {}                         # VSW index -> the parameters of its model, in order
        self._step_tensor = torch.zeros((), dtype=torch.float32)       # Adam's state['step'], shared by all parameters
        self.cos_placeholder = None
        self.grad_placeholders = [[], []]
        workers = self.num_models if self.num_models % 2 == 0 else self.num_models + 1
        self.similarity_state = GradientSimilarityState(None, workers, None, self.grad_placeholders[0], interval)

    # ---------------------------------------------------------------------- set-up
    def prepare_stream_parallel(self, model, criterion, **kwargs):
        """Counterpart of jabas/train/trainer.py:82-86. With a hyperparameter dictionary given to the
        constructor the arenas are built here; otherwise by ``prepare_weight_sync_method``."""
        self._model0 = model.to(self.gpu)
        self.main_model = self._model0
        self.criterion = criterion
        if self.opt is not None:
            self._build(None)

    def prepare_weight_sync_method(self, optimizer, scheduler=None, param_groups_func=None):
        """Counterpart of jabas/train/trainer.py:88-98: takes the optimizer the caller built over
        ``main_model``'s parameters (torch.optim.SGD / Adam / AdamW or ShardSGD / ShardAdam / ShardAdamW,
        examples/resnet50/main.py:351-363) and an optional LR scheduler that is stepped once per sync
        step. Parameter groups of the optimizer become the kernel's parameter groups."""
        if self.main_model is None:
            raise RuntimeError("call prepare_stream_parallel(model, criterion) first")
        if self.engine is not None:
            raise RuntimeError("the weight-sync method is already prepared")
        if param_groups_func is not None:
            self.param_groups_func = param_groups_func
        self.opt = opt_from_torch_optimizer(optimizer)
        self.main_optimizer = optimizer
        self.local_optimizers = [optimizer]          # replicas hold no optimizer state of their own here
        self.local_schedulers = [scheduler] if scheduler is not None else []
        try:
            self._build(optimizer)
        except Exception:                            # leave the trainer as it was: the caller may try again
            self.opt = self.main_optimizer = self.engine = None
            self.local_optimizers, self.local_schedulers = [], []
            raise

    def _build(self, optimizer):
        model = self._model0
        names = [n for n, _ in model.named_parameters()]
        params = [p for _, p in model.named_parameters()]
        group_of = {}
        if optimizer is not None:
            for gi, group in enumerate(optimizer.param_groups):
                for p in group["params"]:
                    group_of[id(p)] = gi
            missing = [n for n, p in zip(names, params) if p.requires_grad and id(p) not in group_of]
            if missing:
                raise ValueError(f"parameters without an optimizer group: {missing[:4]}")
        elif self.param_groups_func is not None:
            for gi, group in enumerate(self.param_groups_func(model)):
                for p in group["params"]:
                    group_of[id(p)] = gi
        specs = [ParamSpec(n, p.numel(), group_of.get(id(p), 0)) for n, p in zip(names, params)]
        # step() clears the buckets right after the update, so the launch need not write the aggregate (nor a
        # clipped step the clipped aggregate) back
        self.engine = VSWFlatSync(specs, self.local_batch_sizes, grad_dtype=self.grad_dtype, opt=self.opt,
                                  device=self.gpu, n_fanout=0 if self.share_weights else max(1, self.num_models - 1),
                                  keep_clipped_grads=self.keep_grads, write_aggregate=self.keep_grads,
                                  moment_block_log2=sync.MOMENT_BLOCK_LOG2 if self.interleave_moments else 0)
        if self.num_models == 1 and not self.share_weights:
            self.engine.reconfigure(self.local_batch_sizes)       # keeps the fan-out slot for later replicas
        self.local_models = [model] + [copy.deepcopy(model) for _ in range(self.num_models - 1)]
        self.main_model = self.local_models[0]
        self.model_streams = [torch.cuda.Stream(self.gpu) for _ in range(self.num_models)]
        for k, m in enumerate(self.local_models):
            self._bind_model(k, m, copy_weights=True)
        if optimizer is not None:
            self._expose_state(optimizer, moments=self.engine.state_is_live)
            if hasattr(optimizer, "register_load_state_dict_post_hook"):
                fresh = not hasattr(optimizer, "_jabas_load_owner")
                optimizer._jabas_load_owner = weakref.ref(self)        # the trainer whose arenas take a loaded state
                if fresh:
                    def adopt(opt):
                        t = opt._jabas_load_owner()
                        if t is not None and t.main_optimizer is opt:
                            t._adopt_optimizer_state()

                    optimizer.register_load_state_dict_post_hook(adopt)
        torch.cuda.synchronize(self.gpu)

    _MOMENT_KEYS = ("exp_avg", "exp_avg_sq", "max_exp_avg_sq")

    def _expose_state(self, optimizer, moments=True):
        """optimizer.state[p] = the state the fused launch maintains under the names torch's optimizers use, so
        that ``state_dict()`` of the caller's optimizer checkpoints it. Flat state arenas: live views. Adam's
        moments interleaved in one arena (the engine's default): they are no flat tensors, so copies are put
        there when the optimizer's ``state_dict()`` is about to read them and taken away again after it
        (hooks registered on the optimizer); in between optimizer.state[p] holds the step count only."""
        eng = self.engine
        sgd = self.opt["kind"] == "sgd"
        for i, p in enumerate(self.main_model.parameters()):
            st = optimizer.state[p]
            if sgd:
                if eng.n_state:
                    st["momentum_buffer"] = eng.state_view(0, i).view(p.shape)
            else:
                st["step"] = self._step_tensor
                for j, key in enumerate(self._MOMENT_KEYS[:eng.n_state]):
                    if moments:
                        st[key] = eng.state_view(j, i).view(p.shape)
                    else:
                        st.pop(key, None)
        if not sgd and not eng.state_is_live:
            hooked = hasattr(optimizer, "_jabas_moment_owner")
            optimizer._jabas_moment_owner = weakref.ref(self)      # the trainer whose arenas the hooks read
            if hooked:
                return

            def owner(opt):
                t = opt._jabas_moment_owner()
                return t if t is not None and t.main_optimizer is opt and t.engine is not None \
                    and not t.engine.state_is_live else None

            def before(opt):
                t = owner(opt)
                if t is not None:
                    torch.cuda.synchronize(t.gpu)
                    t._expose_state(opt, moments=True)

            def after(opt, state_dict):
                t = owner(opt)
                if t is not None:
                    # torch packs the per-parameter dictionaries themselves: the result keeps shallow copies of
                    # them (with the moments), the optimizer's own lose the moments again
                    state_dict["state"] = {idx: dict(st) for idx, st in state_dict["state"].items()}
                    t._expose_state(opt, moments=False)
                return state_dict

            optimizer.register_state_dict_pre_hook(before)
            optimizer.register_state_dict_post_hook(after)

    _adoptions = 0

    def _adopt_optimizer_state(self):
        """After ``main_optimizer.load_state_dict``: the fresh tensors it put into ``optimizer.state`` are copied
        into the arenas the fused launch reads (a parameter the checkpoint holds no state for starts from zeros,
        as it would in torch), the step count follows the checkpoint's (Adam's own count; SGD keeps none, but a
        stored momentum buffer means a step was taken) and the optimizer's dictionaries show the arenas again.
        Runs as a hook on the optimizer, so loading a checkpoint into the caller's optimizer object is enough."""
        eng = self.engine
        if eng is None or self.main_optimizer is None:
            return
        self._adoptions += 1
        torch.cuda.synchronize(self.gpu)
        sgd = self.opt["kind"] == "sgd"
        keys = (("momentum_buffer", 0),) if sgd else tuple((k, j) for j, k in enumerate(self._MOMENT_KEYS))
        steps, has_momentum = set(), False
        for i, p in enumerate(self.main_model.parameters()):
            st = self.main_optimizer.state.get(p, {})
            for key, j in keys:
                if j >= eng.n_state:
                    continue
                loaded = st.get(key)
                if torch.is_tensor(loaded):
                    eng.set_state(j, loaded.to(self.gpu), start=eng.layout.param_offset[i])
                    has_momentum = has_momentum or key == "momentum_buffer"
                else:
                    eng.set_state(j, torch.zeros(p.numel(), dtype=torch.float32, device=self.gpu),
                                  start=eng.layout.param_offset[i])
            if "step" in st:
                steps.add(int(float(st["step"])))
        if len(steps) > 1:
            raise ValueError(f"parameters at different step counts {sorted(steps)}: one fused launch cannot mirror that")
        eng.step_count = steps.pop() if steps else (1 if has_momentum else 0)
        self.opt["groups"] = [dict(lr=float(g["lr"]), weight_decay=float(g.get("weight_decay", 0.0)))
                              for g in self.main_optimizer.param_groups]
        self._step_tensor = torch.full((), float(eng.step_count), dtype=torch.float32)
        self._expose_state(self.main_optimizer, moments=eng.state_is_live)
        torch.cuda.synchronize(self.gpu)

    def _refresh_hyperparameters(self):
        """The hyperparameters as the caller's optimizer object holds them now."""
        if self.main_optimizer is not None:
            refresh_opt_from_torch_optimizer(self.opt, self.main_optimizer)

    def _bind_model(self, k, m, copy_weights):
        """Points replica k's parameters and gradients at its arenas."""
        eng = self.engine
        self._bucket_views.pop(k, None)
        self._params.pop(k, None)
        weights = eng.param if k == 0 or self.share_weights else eng.fanout[k - 1]
        with torch.no_grad():
            for i, p in enumerate(m.parameters()):
                view = eng._view(weights, i).view(p.shape)
                if copy_weights and (k == 0 or not self.share_weights):
                    view.copy_(p.data)
                p.data = view
                p.grad = None

    def _change_local_models_state(self, new_num_models, local_batch_size):
        """Adds or removes VSWs (counterpart of jabas/train/trainer.py:485-575): the engine
        re-plans over the new set, new replicas start from the main weights, weights and
        optimizer state of the main VSW are untouched."""
        torch.cuda.synchronize(self.gpu)
        self.local_batch_sizes = (local_batch_size,) * new_num_models
        self.engine.reconfigure(self.local_batch_sizes)
        while len(self.local_models) < new_num_models:
            self.local_models.append(copy.deepcopy(self.main_model))
            self.model_streams.append(torch.cuda.Stream(self.gpu))
        del self.local_models[new_num_models:]
        del self.model_streams[new_num_models:]
        self._bucket_views.clear()
        self._params.clear()
        for k, m in enumerate(self.local_models):
            self._bind_model(k, m, copy_weights=False)
        self.num_models = self.total_num_decoupled_workers = new_num_models
        workers = new_num_models if new_num_models % 2 == 0 else new_num_models + 1
        self.similarity_state.total_num_decoupled_workers = workers
        self.similarity_state.subgroup_total_num_decoupled_workers = workers / 2
        torch.cuda.synchronize(self.gpu)

    # ---------------------------------------------------------------- checkpoint / resume
    def state_dict(self):
        """What the sync path needs to resume (the reference checkpoints its trainer through
        ``save`` / ``load``, jabas/train/trainer.py:105-170): the main VSW's weights and buffers, the
        optimizer state in torch's own ``Optimizer.state_dict()`` format (so a stock torch optimizer
        can load it, and the other way round), scheduler state, the step counters, the set of VSWs
        and the learning-rate modifier. Tensors are copies, not views of the arenas."""
        if self.engine is None:
            raise RuntimeError("nothing to save before the weight-sync method is prepared")
        torch.cuda.synchronize(self.gpu)
        eng = self.engine
        out = {
            "model": {k: v.detach().clone() for k, v in self.main_model.state_dict().items()},
            "sync_step": self.sync_step,
            "engine_step": eng.step_count,
            "similarity_step": self.similarity_state.step,
            "global_lr_modifier": self.global_lr_modifier,
            "local_batch_sizes": tuple(self.local_batch_sizes),
            "schedulers": [sch.state_dict() for sch in self.local_schedulers],
        }
        if self.main_optimizer is not None:
            sd = self.main_optimizer.state_dict()
            sd["state"] = {idx: {k: (v.detach().clone() if torch.is_tensor(v) else v) for k, v in st.items()}
                           for idx, st in sd["state"].items()}
            out["optimizer"] = sd
        else:
            out["optimizer_arenas"] = {
                "numel": eng.layout.total,
                "state1": None if eng.state1 is None else eng.state1.detach().clone(),
                "state2": None if eng.state2 is None else eng.state2.detach().clone(),
                "state3": None if eng.state3 is None else eng.state3.detach().clone(),
                "groups": [dict(g) for g in self.opt["groups"]],
            }
        return out

    def load_state_dict(self, state):
        """Resumes from ``state_dict()`` (or from a dictionary with the ``model`` and ``optimizer``
        entries of a plain torch training run). Weights and optimizer state are copied into the
        arenas, every replica restarts from the main weights, and the set of VSWs follows the saved
        one. The next step continues bit for bit where the saved run would have."""
        if self.engine is None:
            raise RuntimeError("prepare the weight-sync method before loading a checkpoint")
        torch.cuda.synchronize(self.gpu)
        saved_batches = tuple(state.get("local_batch_sizes", self.local_batch_sizes))
        if saved_batches != tuple(self.local_batch_sizes):
            if len(set(saved_batches)) != 1:
                raise ValueError(f"cannot resume onto unequal local batch sizes {saved_batches}")
            self._change_local_models_state(len(saved_batches), saved_batches[0])
        eng = self.engine
        for m in self.local_models:                     # in-place copies: the parameters stay views of the arenas
            m.load_state_dict(state["model"])
        if "optimizer" in state:
            if self.main_optimizer is None:
                raise ValueError("the checkpoint holds a torch optimizer's state; hand the optimizer over through "
                                 "prepare_weight_sync_method first")
            adopted = self._adoptions
            self.main_optimizer.load_state_dict(state["optimizer"])     # fresh tensors in optimizer.state ...
            if self._adoptions == adopted:                              # ... copied into the arenas (by the hook on
                self._adopt_optimizer_state()                           # the optimizer where torch has such hooks)
            if "engine_step" in state and int(state["engine_step"]) != eng.step_count:
                eng.step_count = int(state["engine_step"])
                self._step_tensor = torch.full((), float(eng.step_count), dtype=torch.float32)
                self._expose_state(self.main_optimizer, moments=eng.state_is_live)
        elif "optimizer_arenas" in state:
            arenas = state["optimizer_arenas"]
            if arenas["numel"] != eng.layout.total:
                raise ValueError("the checkpoint's state arenas belong to another layout")
            for j, theirs in enumerate((arenas["state1"], arenas["state2"], arenas.get("state3"))):
                if (j < eng.n_state) != (theirs is not None):
                    raise ValueError("the checkpoint's optimizer keeps other state than this one")
                if theirs is not None:
                    eng.set_state(j, theirs.to(self.gpu))
            for mine, theirs in zip(self.opt["groups"], arenas["groups"]):
                mine.update(theirs)
            eng.step_count = int(state.get("engine_step", 0))
        for sch, sd in zip(self.local_schedulers, state.get("schedulers", [])):
            sch.load_state_dict(sd)
        self.sync_step = int(state.get("sync_step", eng.step_count))
        self.similarity_state.step = int(state.get("similarity_step", self.sync_step))
        self.global_lr_modifier = float(state.get("global_lr_modifier", 1.0))
        self.accumulated = 0
        for g in eng.grads:
            g.zero_()
        torch.cuda.synchronize(self.gpu)

    # ------------------------------------------------------------------- one iteration
    def compute(self, data):
        """data: one (input, target) pair per VSW, already on the GPU. May be called several times
        before ``step`` (gradient accumulation, IIDP's accum_step): every call adds one micro-batch
        gradient per VSW to its buckets, and the step divides by the number of calls."""
        if len(data) != self.num_models:
            raise ValueError(f"expected {self.num_models} local batches, got {len(data)}")
        cur = torch.cuda.current_stream(self.gpu)
        losses = []
        if self.keep_grads and self.accumulated == 0:
            for p in self._params.get(0, ()):            # the last step's synchronised gradient: backward must not add to it
                p.grad = None
        for k, ((x, y), m, s) in enumerate(zip(data, self.local_models, self.model_streams)):
            s.wait_stream(cur)
            with torch.cuda.stream(s):
                loss = self.criterion(m(x), y)
                loss.backward()
                # The gradients autograd left go into VSW k's bucket views with one multi-tensor launch (rounded
                # there for reduced-precision buckets), and .grad is dropped again: with .grad unset autograd
                # hands over the buffer its backward kernel wrote instead of adding it into an existing tensor
                # with one small kernel per parameter, and the buckets need no clearing between steps (the first
                # micro-batch of a step overwrites them). Per element and VSW that is one read and one write
                # instead of a clearing write plus a read-modify-write.
                params = self._params.get(k)
                if params is None:
                    params = self._params[k] = list(m.parameters())
                    self._bucket_views[k] = [self.engine.grad_view(k, i).view(p.shape) for i, p in enumerate(params)]
                views = self._bucket_views[k]
                have = [(v, p.grad) for v, p in zip(views, params) if p.grad is not None]
                unused = [v for v, p in zip(views, params) if p.grad is None]
                if have:
                    dst, src = [v for v, _ in have], [g for _, g in have]
                    if self.accumulated == 0:
                        torch._foreach_copy_(dst, src)
                    elif self.grad_dtype == torch.float32:
                        torch._foreach_add_(dst, src)
                    else:
                        torch._foreach_add_(dst, [g.to(self.grad_dtype) for g in src])
                if unused and self.accumulated == 0:       # parameters this micro-batch did not reach
                    torch._foreach_zero_(unused)
                for p in params:
                    p.grad = None
                losses.append(loss.detach())
        self.accumulated += 1
        return losses

    def step(self):
        cur = torch.cuda.current_stream(self.gpu)
        for s in self.model_streams:
            cur.wait_stream(s)
        st = self.similarity_state
        want = st.step % st.interval == 0
        self._refresh_hyperparameters()
        # the cosine (and the clipping norm) read the four similarity sums only
        rows = self.engine.step(stats="similarity" if want else False, lr_scale=self.global_lr_modifier, clip_norm=self.clip_norm,
                                accumulations=max(1, self.accumulated))
        self.accumulated = 0
        self.sync_step += 1
        if self.keep_grads:
            for i, p in enumerate(self._params.get(0) or list(self.main_model.parameters())):
                p.grad = self.engine.agg_view(i).view(p.shape)
        self._step_tensor.fill_(float(self.engine.step_count))
        if self.local_schedulers:
            self.main_optimizer._opt_called = True      # what torch's schedulers look at to see that an update preceded them
            for sched in self.local_schedulers:
                sched.step()
        if want:
            self._compute_cosine_similarity(rows)
        for s in self.model_streams:
            s.wait_stream(cur)
        if want and self.controller is not None:
            self._adjust_adaptive_global_batch_size()
        st.step += 1
        return True

    def _adjust_adaptive_global_batch_size(self):
        """jabas/train/trainer.py:702-718: new global batch size from the similarity, the
        matching number of VSWs, and the square-root LR modifier for the following steps."""
        workers, modifier = self.controller.update(float(self.cos_placeholder), step=self.similarity_state.step)
        self.global_lr_modifier = modifier
        if workers != self.num_models:
            self._change_local_models_state(workers, self.controller.local_batch_size)

    def _compute_cosine_similarity(self, rows):
        self.cos_placeholder = torch.tensor([sync.cosine_from_stats(rows)])
        self.similarity_state.grad_placeholder = []
        return self.cos_placeholder
