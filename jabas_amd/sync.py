"""Host side of the fused gradient-sync step: argument marshalling over the C ABI.

Nothing here computes on tensors; every function ends in a libjabas_sync.so call queued
on the current HIP stream. torch is used for device memory and streams only.

Vocabulary: a *span* is one contiguous stretch of the flat layout (normally one DDP
bucket) for which K gradient buffers, the aggregated-gradient output and the parameter /
optimizer-state buffers are indexed alike; a *plan* is a launch-invariant table of spans.
"""
import ctypes as C

import numpy as np
import torch

from . import _lib as L


# ----------------------------------------------------------------------------- weights
def batch_weights(batches, half_id=None, accumulations=1):
    """Per-VSW fp32 weights of the batch-weighted aggregate and of the two halves.

    w_k = fp32(b_k / B): the quotient is formed in double and rounded once, which is what
    a Python float becomes when ATen applies it to an fp32 tensor. Halves follow the
    reference's rank-parity split (jabas/train/trainer.py:427-432) mapped onto the VSW
    index: even k -> half A (0), odd k -> half B (1).

    ``accumulations``: micro-batches each VSW accumulated into its bucket before this sync step
    (IIDP's accum_step + 1). The bucket then holds a sum of that many mean gradients, and the
    reference's divisor, the number of decoupled workers, counts them
    (jabas/train/trainer.py:594-599: global batch = local batch x decoupled workers), so
    w_k = fp32(b_k / (B * accumulations)).
    """
    if int(accumulations) < 1:
        raise ValueError("accumulations must be a positive integer")
    b = [float(x) for x in batches]
    K = len(b)
    if not 1 <= K <= L.MAX_K:
        raise ValueError(f"number of VSWs must be in 1..{L.MAX_K}, got {K}")
    if any(x <= 0 for x in b):
        raise ValueError(f"local batch sizes must be positive: {batches}")
    acc = float(int(accumulations))
    total = sum(b) * acc
    w = np.array([x / total for x in b], dtype=np.float64).astype(np.float32)
    if half_id is None:
        half_id = [k % 2 for k in range(K)]
    half_id = np.array(half_id, dtype=np.uint8)
    if half_id.shape != (K,) or np.any(half_id > 1):
        raise ValueError("half_id must hold K entries of 0 or 1")
    hw = np.zeros(K, dtype=np.float32)
    for h in (0, 1):
        tot = sum(x for x, hid in zip(b, half_id) if hid == h) * acc
        for k in range(K):
            if half_id[k] == h:
                hw[k] = np.float32(b[k] / tot)
    return w, half_id, hw


_KIND = {None: L.OPT_NONE, "none": L.OPT_NONE, "sgd": L.OPT_SGD, "adam": L.OPT_ADAM, "adamw": L.OPT_ADAMW}


def opt_kind(opt):
    """JABAS_OPT_* code of a hyperparameter dictionary; ``amsgrad=True`` selects the Adam / AdamW kinds that
    keep the running maximum of the second moment (``state3`` of the spans)."""
    kind = None if opt is None else opt["kind"]
    if kind not in _KIND:
        raise ValueError(f"unknown optimizer kind {kind!r}")
    if opt is not None and opt.get("amsgrad", False):
        if kind not in ("adam", "adamw"):
            raise ValueError("amsgrad belongs to Adam and AdamW")
        return L.OPT_ADAMW_AMSGRAD if kind == "adamw" else L.OPT_ADAM_AMSGRAD
    return _KIND[kind]


def stats_level(stats):
    """JABAS_STATS_* level of a launch: False / None / 0 none; True / 1 / 'full' the full row (4 + K sums);
    2 / 'similarity' the four sums of the halves and of the aggregate only (what the cosine similarity and
    global-norm clipping read; the per-VSW norm slots of the row are 0); 3 / 'gram' the full row plus the
    products of every pair of workers (the Gram matrix out of the same pass; up to STATS_GRAM_MAX_K workers;
    read it with :func:`gram_from_stats`)."""
    if stats is None or stats is False or stats == 0:
        return L.STATS_NONE
    if stats is True or stats == 1 or stats == "full":
        return L.STATS_FULL
    if stats == 2 or stats == "similarity":
        return L.STATS_SIMILARITY
    if stats == 3 or stats == "gram":
        return L.STATS_GRAM
    raise ValueError(f"unknown statistics level {stats!r}")


def grad_dtype_code(dtype):
    if dtype == torch.float32:
        return L.F32
    if dtype == torch.bfloat16:
        return L.BF16
    raise TypeError(f"gradient dtype must be float32 or bfloat16, got {dtype}")


def make_step_args(batches, grad_dtype, stats=False, opt=None, step=1, first_step=False, half_id=None,
                   lr_scale=1.0, grad_scale=None, accumulations=1):
    """Builds the JabasStepArgs of one call.

    ``opt``: None or dict(kind='sgd'|'adam'|'adamw', groups=[dict(lr=, weight_decay=)], plus
    momentum/dampening/nesterov or betas/eps). ``step`` is the 1-based Adam step count,
    ``lr_scale`` the adaptive-batching LR modifier (jabas/train/trainer.py:693-700).
    """
    w, hid, hw = batch_weights(batches, half_id, accumulations)
    a = L.JabasStepArgs()
    a.K = len(w)
    a.grad_dtype = grad_dtype_code(grad_dtype)
    for k in range(a.K):
        a.weight[k] = float(w[k])
        a.half_id[k] = int(hid[k])
        a.half_weight[k] = float(hw[k])
    a.stats = stats_level(stats)
    a.opt_kind = opt_kind(opt)
    if opt is not None and a.opt_kind != L.OPT_NONE:
        groups = opt["groups"]
        if not 1 <= len(groups) <= L.MAX_GROUPS:
            raise ValueError(f"1..{L.MAX_GROUPS} parameter groups supported, got {len(groups)}")
        a.n_groups = len(groups)
        for i, g in enumerate(groups):
            a.groups[i].lr = float(g["lr"]) * float(lr_scale)
            a.groups[i].weight_decay = float(g.get("weight_decay", 0.0))
            a.groups[i].step = int(g.get("step", step))
        a.first_step = 1 if first_step else 0
        a.nesterov = 1 if opt.get("nesterov", False) else 0
        a.momentum = float(opt.get("momentum", 0.0))
        a.dampening = float(opt.get("dampening", 0.0))
        b1, b2 = opt.get("betas", (0.9, 0.999))
        a.beta1, a.beta2 = float(b1), float(b2)
        a.eps = float(opt.get("eps", 1e-8))
    if grad_scale is not None:
        if grad_scale.dtype != torch.float32 or not grad_scale.is_cuda:
            raise TypeError("grad_scale must be an fp32 scalar on the GPU")
        a.grad_scale = grad_scale.data_ptr()
        a._keep_grad_scale = grad_scale          # keeps the tensor alive as long as the args
    return a


class StepScalars:
    """The scalars of a step that move from step to step (weights, learning rates, Adam's bias corrections,
    the first-step flag) as a block in device memory, for launches recorded in a HIP graph: a recorded launch
    has its by-value arguments baked in, one that names this block (``attach``) reads the block as it is when
    the kernel runs. ``update(args)`` encodes the arguments of the coming step on the host (the same
    double -> fp32 derivation as a plain call) and queues a one-wave kernel that writes them to the block
    (``jabas_step_scalars_upload``), on the stream the replay follows on."""

    def __init__(self, device):
        self.dev = torch.zeros(L.STEP_SCALARS_BYTES, dtype=torch.uint8, device=device)

    def attach(self, args):
        args.scalars_dev = self.dev.data_ptr()
        args._keep_scalars = self                   # keeps the block alive as long as the args
        return args

    def update(self, args, stream=None):
        L.check(L.lib().jabas_step_scalars_upload(C.byref(args), self.dev.data_ptr(), _stream_ptr(stream)),
                "jabas_step_scalars_upload")


# ------------------------------------------------------------------------------- spans
def _ptr(t):
    return None if t is None else t.data_ptr()


def _check_tensor(t, n, dtype, what, device):
    if t is None:
        return
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what}: expected a tensor")
    if t.dtype != dtype:
        raise TypeError(f"{what}: expected {dtype}, got {t.dtype}")
    if t.device != device:
        raise ValueError(f"{what}: on {t.device}, expected {device}")
    if not t.is_contiguous() or t.numel() != n:
        raise ValueError(f"{what}: must be contiguous with {n} elements (has {t.numel()})")


MOMENT_BLOCK_LOG2 = 13      # 8192 elements, 32 KiB: with 16384 the fastest block size measured (2048 ... 131072)


class MomentArena:
    """Adam's moments of ``numel`` elements in ONE device buffer that alternates blocks of T = 2**block_log2
    elements of exp_avg and of exp_avg_sq (``ways=3``: and of max_exp_avg_sq, amsgrad):
    [T of exp_avg][T of exp_avg_sq]... The moments are state only the optimizer touches, so their place in HBM
    is free to choose, and the fused kernels stream this layout 2-6 % faster than arrays of their own: what a
    workgroup reads and writes of the moments lies together in memory (``JabasSpan.state_block_log2``).

    Element i of moment j sits at float index i + (ways - 1) * (i - i % T) + j * T of ``buf``. A moment is
    therefore not a flat tensor: ``way(j)`` is its (blocks, T) strided view, ``read`` / ``write`` copy a flat
    range out of it or into it (checkpoints, tests)."""

    def __init__(self, numel, ways, device, block_log2=MOMENT_BLOCK_LOG2):
        if ways not in (2, 3):
            raise ValueError("two moments (Adam, AdamW) or three (amsgrad)")
        if not 8 <= int(block_log2) <= 24:
            raise ValueError("blocks of 2**8 to 2**24 elements")
        self.numel, self.ways, self.block_log2 = int(numel), ways, int(block_log2)
        self.T = 1 << self.block_log2
        self.blocks = max(1, -(-self.numel // self.T))
        raw = torch.zeros(self.blocks * ways * self.T + 64, dtype=torch.float32, device=device)
        skip = (-(raw.data_ptr() // 4)) % 64                      # block groups start on 256-byte lines
        self.buf = raw[skip:skip + self.blocks * ways * self.T]
        self._view = self.buf.view(self.blocks, ways, self.T)

    @property
    def device(self):
        return self.buf.device

    def way(self, j):
        """(blocks, T) strided view of moment j (0 exp_avg, 1 exp_avg_sq, 2 max_exp_avg_sq)."""
        return self._view[:, j, :]

    def read(self, j, start=0, count=None):
        """Contiguous copy of elements [start, start + count) of moment j."""
        count = self.numel - start if count is None else count
        if count <= 0:
            return torch.empty(0, dtype=torch.float32, device=self.device)
        b0, b1 = start // self.T, (start + count - 1) // self.T + 1
        lo = start - b0 * self.T
        if b1 - b0 == 1:
            return self._view[b0, j, lo:lo + count].clone()
        return self._view[b0:b1, j, :].reshape(-1)[lo:lo + count]

    def write(self, j, values, start=0):
        """Copies the flat tensor ``values`` into elements [start, start + values.numel()) of moment j."""
        values = values.reshape(-1)
        count = values.numel()
        if count == 0:
            return
        if start < 0 or start + count > self.blocks * self.T:
            raise ValueError("range outside the arena")
        b0, b1 = start // self.T, (start + count - 1) // self.T + 1
        lo = start - b0 * self.T
        if b1 - b0 == 1:                                         # inside one block: contiguous in the arena
            self._view[b0, j, lo:lo + count].copy_(values)
            return
        sub = self._view[b0:b1, j, :]
        flat = sub.reshape(-1)                                   # a copy: the view is strided
        flat[lo:lo + count] = values.to(flat.dtype)
        sub.copy_(flat.view(b1 - b0, self.T))

    def zero_(self):
        self.buf.zero_()
        return self

    def place(self, first):
        """(address of element ``first``'s exp_avg, its position in its block): what a span that starts at
        arena element ``first`` names as state1 and state_block_pos."""
        pos = first % self.T
        return self.buf.data_ptr() + 4 * ((first // self.T) * self.ways * self.T + pos), pos


class SpanSpec:
    """Tensors of one span. All 1-D (or contiguous) with the same number of elements. ``moments=(arena,
    first)``: Adam's moments of the span are elements [first, first + n) of a ``MomentArena`` instead of the
    tensors state1 / state2 / state3."""

    def __init__(self, grads, agg_out=None, param=None, state1=None, state2=None, fanout=(), bounds=(), state3=None,
                 moments=None):
        self.grads = list(grads)
        self.agg_out, self.param, self.state1, self.state2, self.state3 = agg_out, param, state1, state2, state3
        self.fanout = list(fanout)
        self.bounds = list(bounds)          # [(start_element, group), ...], first start 0
        self.moments = moments
        if moments is not None and (state1 is not None or state2 is not None or state3 is not None):
            raise ValueError("moments= stands for state1, state2 and state3: pass one or the other")

    def validate(self):
        if not self.grads:
            raise ValueError("a span needs at least one gradient buffer")
        g0 = self.grads[0]
        n, dev, gdt = g0.numel(), g0.device, g0.dtype
        if dev.type != "cuda":
            raise ValueError(f"gradient buffers must live on the GPU, got {dev}")
        for k, g in enumerate(self.grads):
            _check_tensor(g, n, gdt, f"grads[{k}]", dev)
        _check_tensor(self.agg_out, n, torch.float32, "agg_out", dev)
        _check_tensor(self.param, n, torch.float32, "param", dev)
        _check_tensor(self.state1, n, torch.float32, "state1", dev)
        _check_tensor(self.state2, n, torch.float32, "state2", dev)
        _check_tensor(self.state3, n, torch.float32, "state3", dev)
        for r, f in enumerate(self.fanout):
            _check_tensor(f, n, torch.float32, f"fanout[{r}]", dev)
        if self.moments is not None:
            arena, first = self.moments
            if arena.device != dev:
                raise ValueError(f"the moment arena lives on {arena.device}, the span on {dev}")
            if first < 0 or first + n > arena.blocks * arena.T:
                raise ValueError("the span's elements lie outside the moment arena")
        return n, dev, gdt

    def to_c(self, bound_begin=0):
        n, _, _ = self.validate()
        s = L.JabasSpan()
        for k, g in enumerate(self.grads):
            s.grads[k] = g.data_ptr()
        s.agg_out = _ptr(self.agg_out)
        s.param = _ptr(self.param)
        if self.moments is not None:
            arena, first = self.moments
            s.state1, s.state_block_pos = arena.place(first)
            s.state2 = s.state1 + 4 * arena.T
            s.state3 = s.state1 + 8 * arena.T if arena.ways == 3 else None
            s.state_block_log2 = arena.block_log2
        else:
            s.state1 = _ptr(self.state1)
            s.state2 = _ptr(self.state2)
            s.state3 = _ptr(self.state3)
        for r, f in enumerate(self.fanout):
            s.fanout[r] = f.data_ptr()
        s.numel = n
        s.n_fanout = len(self.fanout)
        s.bound_begin = bound_begin
        s.bound_count = len(self.bounds)
        return s


def _bounds_array(bounds):
    arr = (L.JabasBound * max(1, len(bounds)))()
    for i, (start, group) in enumerate(bounds):
        arr[i].start = int(start)
        arr[i].group = int(group)
    return arr


def _stream_ptr(stream=None):
    s = torch.cuda.current_stream() if stream is None else stream
    return C.c_void_p(s.cuda_stream)


class Workspace:
    """Device scratch of the two-level statistics reduction plus the stats rows.

    ``Workspace.for_span(numel, dtype, device)`` sizes it for single-span calls over up to
    ``numel`` elements; plans size their own."""

    def __init__(self, nbytes, n_span, device):
        self.buf = torch.empty(max(1, nbytes // 8), dtype=torch.float64, device=device)
        self.nbytes = nbytes
        self.stats = torch.zeros(n_span, L.STATS_STRIDE, dtype=torch.float64, device=device)

    @classmethod
    def for_span(cls, numel, grad_dtype, device):
        return cls(L.lib().jabas_sync_workspace_bytes(int(numel), grad_dtype_code(grad_dtype)), 1, device)


class SyncPlan:
    """A validated, device-resident table of spans; ``run`` queues the fused step."""

    def __init__(self, spans, opt_kind_code=L.OPT_NONE):
        lib = L.lib()
        self.spans = list(spans)
        if not self.spans:
            raise ValueError("a plan needs at least one span")
        n0, dev, gdt = self.spans[0].validate()
        self.device, self.grad_dtype = dev, gdt
        self.K = len(self.spans[0].grads)
        self.opt_kind = opt_kind_code
        n_span = len(self.spans)
        c_spans = (L.JabasSpan * n_span)()
        all_bounds = []
        for i, sp in enumerate(self.spans):
            _, d, t = sp.validate()
            if d != dev or t != gdt or len(sp.grads) != self.K:
                raise ValueError(f"span {i}: device, gradient dtype or K differs from span 0")
            c_spans[i] = sp.to_c(bound_begin=len(all_bounds))
            all_bounds += sp.bounds
        c_bounds = _bounds_array(all_bounds)
        nbytes = lib.jabas_plan_bytes(c_spans, n_span, len(all_bounds), grad_dtype_code(gdt))
        self._host = np.zeros((nbytes + 7) // 8, dtype=np.uint64)        # 8-byte aligned blob
        L.check(lib.jabas_plan_encode(c_spans, n_span, c_bounds if all_bounds else None, len(all_bounds),
                                      self.K, grad_dtype_code(gdt), opt_kind_code,
                                      self._host.ctypes.data, nbytes), "jabas_plan_encode")
        self.n_chunks = int(lib.jabas_plan_chunks(self._host.ctypes.data, 0))            # workgroups of a plain launch
        self.n_chunks_stats = int(lib.jabas_plan_chunks(self._host.ctypes.data, 1))      # of a launch with full statistics rows
        self.n_chunks_similarity = int(lib.jabas_plan_chunks(self._host.ctypes.data, 2)) # of a launch with similarity sums
        self._dev = torch.from_numpy(self._host.view(np.int64)).to(dev)
        self.ws = Workspace(lib.jabas_plan_workspace_bytes(self._host.ctypes.data), n_span, dev)
        self.n_span = n_span

    def run(self, args, stream=None):
        """Queues aggregate (+stats, +optimizer) over every span. Returns the stats tensor
        (n_span x STATS_STRIDE doubles, device) when args.stats is set, else None."""
        L.check(L.lib().jabas_sync_fused(self._host.ctypes.data, self._dev.data_ptr(), C.byref(args),
                                         self.ws.stats.data_ptr() if args.stats else None,
                                         self.ws.buf.data_ptr(), self.ws.nbytes, _stream_ptr(stream)),
                "jabas_sync_fused")
        return self.ws.stats if args.stats else None


# ------------------------------------------------------------- single-bucket entry points
def sync_bucket(span, args, workspace=None, bounds_dev=None, stream=None):
    """One span by value (what a comm hook calls for the bucket it was handed)."""
    c_span = span.to_c()
    if span.bounds and bounds_dev is None:
        bounds_dev = bounds_to_device(span.bounds, span.grads[0].device)
    stats_ptr = ws_ptr = None
    ws_bytes = 0
    if args.stats:
        if workspace is None:
            workspace = Workspace.for_span(span.grads[0].numel(), span.grads[0].dtype, span.grads[0].device)
        stats_ptr, ws_ptr, ws_bytes = workspace.stats.data_ptr(), workspace.buf.data_ptr(), workspace.nbytes
    L.check(L.lib().jabas_sync_bucket(C.byref(c_span), None if bounds_dev is None else bounds_dev.data_ptr(),
                                      C.byref(args), stats_ptr, ws_ptr, ws_bytes, _stream_ptr(stream)),
            "jabas_sync_bucket")
    if stream is not None:                          # temporaries made here are freed on return: the allocator
        for t in (bounds_dev, workspace and workspace.buf, workspace and workspace.stats):   # must know who uses them
            if t is not None:
                t.record_stream(stream)
    return workspace.stats[0] if args.stats else None


def sync_bucket_static(span, args, stats_out=None, bounds_dev=None, stream=None):
    """``jabas_sync_bucket_static``: one span by value with the statistics scratch in the library's static
    device array (no workspace, nothing allocated by the call). ``stats_out``: caller-owned device row of
    STATS_STRIDE doubles, required when args.stats is set; ``bounds_dev``: device bound table from
    ``bounds_to_device`` when the span has bounds. Calls with statistics on one GPU must not overlap."""
    c_span = span.to_c()
    if span.bounds and bounds_dev is None:
        raise ValueError("pass the span's bound table on the device (bounds_to_device): this call allocates nothing")
    if args.stats and stats_out is None:
        raise ValueError("pass stats_out: this call allocates nothing")
    L.check(L.lib().jabas_sync_bucket_static(C.byref(c_span), None if bounds_dev is None else bounds_dev.data_ptr(),
                                             C.byref(args), None if stats_out is None else stats_out.data_ptr(),
                                             _stream_ptr(stream)), "jabas_sync_bucket_static")
    return stats_out


def bounds_to_device(bounds, device):
    """Device copy of a span's bound table in JabasBound layout (for ``jabas_sync_bucket``)."""
    host = np.zeros((len(bounds), 2), dtype=np.uint64)
    for i, (start, group) in enumerate(bounds):
        host[i, 0] = start
        host[i, 1] = group                          # low 32 bits = group, high 32 = reserved
    return torch.from_numpy(host.view(np.int64)).to(device)


class BucketCall:
    """One span prepared for repeated ``jabas_sync_bucket`` calls: the tensors are validated, the
    C struct is filled, the bound table is on the device and the statistics workspace exists, so that
    ``run`` is one foreign call. A comm hook sees the same bucket buffers every step; ``matches``
    tells whether a prepared call still describes them."""

    def __init__(self, span):
        self.span = span
        self.c_span = span.to_c()
        g0 = span.grads[0]
        self.key = self.key_of(span.grads)
        self.bounds_dev = bounds_to_device(span.bounds, g0.device) if span.bounds else None
        self.ws = None                              # created by the first statistics launch
        self._fn = L.lib().jabas_sync_bucket

    @staticmethod
    def key_of(grads):
        return tuple(g.data_ptr() for g in grads) + (grads[0].numel(),)

    def matches(self, grads):
        return self.key == self.key_of(grads)

    def prepare_stats(self):
        """The statistics workspace and the two rows the launches alternate between (made once)."""
        if self.ws is None:
            g0 = self.span.grads[0]
            self.ws = Workspace.for_span(g0.numel(), g0.dtype, g0.device)
            self._rows = torch.zeros(2, L.STATS_STRIDE, dtype=torch.float64, device=g0.device)
            self._flip = 0

    def run(self, args, stream=None):
        """Queues the step; returns the statistics row or None. Rows alternate between two device
        buffers, so a returned row stays untouched by this call's next statistics launch and is
        overwritten by the one after that."""
        stats_ptr = ws_ptr = row = None
        ws_bytes = 0
        if args.stats:
            self.prepare_stats()
            self._flip ^= 1
            row = self._rows[self._flip]
            stats_ptr, ws_ptr, ws_bytes = row.data_ptr(), self.ws.buf.data_ptr(), self.ws.nbytes
        L.check(self._fn(C.byref(self.c_span), None if self.bounds_dev is None else self.bounds_dev.data_ptr(),
                         C.byref(args), stats_ptr, ws_ptr, ws_bytes, _stream_ptr(stream)), "jabas_sync_bucket")
        return row


def _ptr_array(tensors):
    arr = (C.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def aggregate(grads, batches, out=None, stream=None):
    """out = sum_k w_k g_k (canonical order); ``out`` may be grads[0] for fp32 gradients."""
    span = SpanSpec(grads)
    n, dev, gdt = span.validate()
    if out is None:
        out = torch.empty(n, dtype=torch.float32, device=dev)
    _check_tensor(out, n, torch.float32, "out", dev)
    w, _, _ = batch_weights(batches)
    if len(w) != len(grads):
        raise ValueError("one batch size per gradient buffer")
    cw = (C.c_float * len(w))(*[float(x) for x in w])
    L.check(L.lib().jabas_aggregate(_ptr_array(grads), len(grads), grad_dtype_code(gdt), cw, out.data_ptr(), n,
                                    _stream_ptr(stream)), "jabas_aggregate")
    return out


def gradient_stats(grads, batches, half_id=None, workspace=None, stream=None):
    """Statistics row (STATS_STRIDE doubles, device) of one span; writes nothing else."""
    span = SpanSpec(grads)
    n, dev, gdt = span.validate()
    w, hid, hw = batch_weights(batches, half_id)
    if len(w) != len(grads):
        raise ValueError("one batch size per gradient buffer")
    if workspace is None:
        workspace = Workspace.for_span(n, gdt, dev)
    K = len(w)
    L.check(L.lib().jabas_stats(_ptr_array(grads), K, grad_dtype_code(gdt),
                                (C.c_float * K)(*[float(x) for x in w]),
                                (C.c_uint8 * K)(*[int(x) for x in hid]),
                                (C.c_float * K)(*[float(x) for x in hw]), n,
                                workspace.stats.data_ptr(), workspace.buf.data_ptr(), workspace.nbytes,
                                _stream_ptr(stream)), "jabas_stats")
    if stream is not None:
        workspace.buf.record_stream(stream)
        workspace.stats.record_stream(stream)
    return workspace.stats[0]


def gram(grads, stream=None, workspace=None):
    """K x K Gram matrix (float64, device) of the worker gradients. ``workspace``: a float64 device tensor of
    at least 1024 * GRAM_STRIDE elements (1056 * GRAM_STRIDE for the faster two-stage sum of the partial rows);
    allocated per call when None."""
    span = SpanSpec(grads)
    n, dev, gdt = span.validate()
    K = len(grads)
    if workspace is None:
        ws = torch.empty(1056 * L.GRAM_STRIDE, dtype=torch.float64, device=dev)
    else:
        ws = workspace
        if ws.dtype != torch.float64 or ws.device != dev or not ws.is_contiguous():
            raise ValueError("workspace must be a contiguous float64 tensor on the gradients' device")
    out = torch.empty(L.GRAM_STRIDE, dtype=torch.float64, device=dev)
    L.check(L.lib().jabas_gram(_ptr_array(grads), K, grad_dtype_code(gdt), n, out.data_ptr(), ws.data_ptr(),
                               ws.numel() * 8, _stream_ptr(stream)), "jabas_gram")
    if stream is not None:
        ws.record_stream(stream)
        out.record_stream(stream)
    return out.view(L.GRAM_MAX_K, L.GRAM_MAX_K)[:K, :K]


def gram_from_stats(stats_rows, K):
    """K x K Gram matrix (float64, on the rows' device) of the worker gradients from statistics rows of level
    'gram', summed over the rows (one row per span or bucket): the diagonal from the per-VSW norms, the rest
    from the pair slots. No launch of its own: the sums came out of the pass that aggregated the gradients."""
    if not 1 <= K <= L.STATS_GRAM_MAX_K:
        raise ValueError(f"rows of level 'gram' exist for 1..{L.STATS_GRAM_MAX_K} workers, not {K}")
    total = stats_rows.detach().reshape(-1, L.STATS_STRIDE).to(torch.float64).sum(dim=0)
    out = torch.empty(K, K, dtype=torch.float64, device=total.device)
    for a in range(K):
        out[a, a] = total[L.STAT_NORM_VSW0 + a]
        for b in range(a + 1, K):
            out[a, b] = out[b, a] = total[L.stat_pair(K, a, b)]
    return out


def sgd_step(grad, param, momentum_buf, lr, weight_decay=0.0, momentum=0.0, dampening=0.0, nesterov=False,
             first_step=False, stream=None):
    n = param.numel()
    _check_tensor(grad, n, torch.float32, "grad", param.device)
    _check_tensor(momentum_buf, n, torch.float32, "momentum_buf", param.device)
    L.check(L.lib().jabas_sgd(grad.data_ptr(), param.data_ptr(), _ptr(momentum_buf), n, lr, weight_decay, momentum,
                              dampening, int(bool(nesterov)), int(bool(first_step)), _stream_ptr(stream)), "jabas_sgd")


def adam_step(grad, param, exp_avg, exp_avg_sq, lr, weight_decay, betas, eps, step, adamw, stream=None,
              max_exp_avg_sq=None):
    """``max_exp_avg_sq``: the running maximum of the second moment: the step is then amsgrad's."""
    n = param.numel()
    for t, what in ((grad, "grad"), (exp_avg, "exp_avg"), (exp_avg_sq, "exp_avg_sq"), (max_exp_avg_sq, "max_exp_avg_sq")):
        _check_tensor(t, n, torch.float32, what, param.device)
    L.check(L.lib().jabas_adam(grad.data_ptr(), param.data_ptr(), exp_avg.data_ptr(), exp_avg_sq.data_ptr(),
                               _ptr(max_exp_avg_sq), n,
                               lr, weight_decay, betas[0], betas[1], eps, int(step), int(bool(adamw)),
                               _stream_ptr(stream)), "jabas_adam")


def clip_coef(stats_rows, max_norm, eps=1e-6, out=None, stream=None):
    """Device scalar max_norm / (||aggregate|| + eps) from statistics rows (no host sync);
    pass it as ``grad_scale`` of a later step to clip the aggregate by global norm."""
    rows = stats_rows.reshape(-1, L.STATS_STRIDE)
    if out is None:
        out = torch.empty(1, dtype=torch.float32, device=rows.device)
    L.check(L.lib().jabas_clip_coef(rows.data_ptr(), rows.shape[0], float(max_norm), float(eps), out.data_ptr(),
                                    _stream_ptr(stream)), "jabas_clip_coef")
    return out


# ---------------------------------------------------------------------- cosine similarity
def cosine_from_stats(stats_rows, eps=1e-8):
    """cos(g_A, g_B) over all spans from their statistics rows (host scalars).

    Sums the per-span triples (the reference concatenates the per-bucket tensors instead,
    jabas/train/trainer.py:475) and applies torch 1.8.1's cosine_similarity formula
    dot / sqrt(max(|a|^2 |b|^2, eps^2)).
    """
    rows = stats_rows.detach().to("cpu", torch.float64).reshape(-1, L.STATS_STRIDE)
    dot = float(rows[:, L.STAT_DOT_AB].sum())
    na = float(rows[:, L.STAT_NORM_A].sum())
    nb = float(rows[:, L.STAT_NORM_B].sum())
    return dot / max(na * nb, eps * eps) ** 0.5
