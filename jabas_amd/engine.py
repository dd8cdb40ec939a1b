"""Flat-arena owner of one GPU's gradient-sync state.

``VSWFlatSync`` lays the whole gradient set out MI355X-first: one arena per VSW for the
gradient buckets, one each for the aggregated gradient, the fp32 weights and the
optimizer state, all with the same bucket layout (FlatLayout), so that a whole sync
step is one kernel launch over a device-resident span table instead of the reference's
per-bucket hook plus per-tensor optimizer loop (jabas/train/trainer.py:327-337,
examples/gnmt/seq2seq/train/shard_optimizer.py:40-90). Model code reaches its tensors
through views (``param_view``, ``grad_view``).
"""
import torch

from . import _lib as L
from .layout import FlatLayout
from .sync import SpanSpec, SyncPlan, StepScalars, MomentArena, MOMENT_BLOCK_LOG2, gradient_stats, make_step_args, opt_kind, cosine_from_stats, clip_coef, gram_from_stats


class VSWFlatSync:
    def __init__(self, specs, batches, grad_dtype=torch.float32, opt=None, device="cuda", in_place=None,
                 n_fanout=0, per_tensor_spans=False, caps=None, keep_clipped_grads=True, write_aggregate=True,
                 moment_block_log2=MOMENT_BLOCK_LOG2):
        self.K = len(batches)
        # Adam's moments (exp_avg, exp_avg_sq, amsgrad's maximum) live in ONE arena that alternates blocks of
        # 2**moment_block_log2 elements of each (sync.MomentArena): the kernels stream that 2-6 % faster than
        # arenas of their own. ``state1`` / ``state2`` / ``state3`` then are flat COPIES made on access
        # (``set_state`` writes one back); 0 or None: flat arenas as for SGD's momentum buffer.
        self.moment_block_log2 = int(moment_block_log2 or 0)
        # False: the launch hands the aggregate to the optimizer in registers and writes it nowhere (4 of the
        # 44 bytes per element of an Adam step with four fp32 workers). For owners of the whole step who clear
        # or overwrite the buckets right after it, as the trainer does; a comm hook has to leave the
        # synchronised gradient in the main VSW's bucket and cannot use this. Ignored without optimizer.
        self.write_aggregate = bool(write_aggregate) or opt is None
        # clipped steps: True leaves the clipped aggregate in the gradient arena, as clip_grad_norm_
        # leaves the clipped .grad behind; False saves that write (4 of 52 bytes per element)
        self.keep_clipped_grads = keep_clipped_grads
        self.batches = tuple(batches)
        self.grad_dtype = grad_dtype
        self.opt = opt
        self.device = torch.device(device)
        kw = {} if caps is None else {"caps": caps}
        self.layout = FlatLayout(specs, per_tensor_spans=per_tensor_spans, **kw)
        n = self.layout.total
        # in place: the aggregate overwrites VSW 0's buckets, as the reference's main VSW
        # bucket ends up holding the synchronised gradient
        if in_place is None:
            in_place = grad_dtype == torch.float32
        if in_place and grad_dtype != torch.float32:
            raise ValueError("in-place aggregation needs fp32 gradient buckets")
        self.grads = [torch.zeros(n, dtype=grad_dtype, device=self.device) for _ in range(self.K)]
        self.in_place = bool(in_place)
        if in_place:
            self.agg = self.grads[0]
        else:                                    # an arena of its own, unless nothing will ever be written to it
            self.agg = torch.zeros(n, dtype=torch.float32, device=self.device) if self.write_aggregate else None
        kind = opt_kind(opt)
        self.param = self._state = None
        self.moments = None
        self.fanout = []
        if kind != L.OPT_NONE:
            if len(opt["groups"]) < self.layout.n_groups:
                raise ValueError(f"layout names {self.layout.n_groups} parameter groups, optimizer has "
                                 f"{len(opt['groups'])}")
            self.param = torch.zeros(n, dtype=torch.float32, device=self.device)
            adam = kind in (L.OPT_ADAM, L.OPT_ADAMW, L.OPT_ADAM_AMSGRAD, L.OPT_ADAMW_AMSGRAD)
            ways = 3 if kind in (L.OPT_ADAM_AMSGRAD, L.OPT_ADAMW_AMSGRAD) else 2        # amsgrad: max_exp_avg_sq
            if adam and self.moment_block_log2:
                self.moments = MomentArena(n, ways, self.device, self.moment_block_log2)
            elif adam:
                self._state = [torch.zeros(n, dtype=torch.float32, device=self.device) for _ in range(ways)]
            elif opt.get("momentum", 0.0) != 0.0:
                self._state = [torch.zeros(n, dtype=torch.float32, device=self.device)]
            self.fanout = [torch.zeros(n, dtype=torch.float32, device=self.device) for _ in range(n_fanout)]
        self._fanout_wanted = n_fanout > 0
        self._build_plan()
        self.step_count = 0

    # ---- optimizer state ---------------------------------------------------------
    def _state_arena(self, j):
        if self.moments is not None:
            return self.moments.read(j) if j < self.moments.ways else None
        return self._state[j] if self._state is not None and j < len(self._state) else None

    @property
    def state1(self):
        """SGD's momentum buffer / Adam's exp_avg as a flat fp32 tensor laid out like ``param``: the arena itself
        when the state is kept in flat arenas, a copy made now when the moments are interleaved."""
        return self._state_arena(0)

    @property
    def state2(self):
        return self._state_arena(1)

    @property
    def state3(self):
        return self._state_arena(2)

    def set_state(self, j, values, start=0):
        """Writes the flat tensor ``values`` into elements [start, ...) of state j (0, 1, 2 as state1..3)."""
        if self.moments is not None:
            self.moments.write(j, values, start)
        else:
            self._state[j][start:start + values.numel()].copy_(values.reshape(-1))

    def state_view(self, j, i):
        """State j of parameter i in the parameter's flat order: a live view of a flat arena, a copy when the
        moments are interleaved (``state_is_live`` tells which)."""
        off, n = self.layout.param_offset[i], self.layout.specs[i].numel
        if self.moments is not None:
            return self.moments.read(j, off, n)
        return self._state[j][off:off + n]

    @property
    def state_is_live(self):
        return self.moments is None

    @property
    def n_state(self):
        """State arrays the optimizer keeps per element: 0 (none, SGD without momentum), 1, 2 or 3 (amsgrad)."""
        return self.moments.ways if self.moments is not None else len(self._state or [])

    def state_of_span(self, off, numel):
        """SpanSpec keywords naming the optimizer state of arena elements [off, off + numel)."""
        if self.moments is not None:
            return dict(moments=(self.moments, off))
        st = self._state or []
        names = ("state1", "state2", "state3")
        return {names[j]: st[j][off:off + numel] for j in range(len(st))}

    def _build_plan(self):
        kind = opt_kind(self.opt)
        spans = []
        for (off, numel, bounds, _bucket) in self.layout.spans:
            sl = slice(off, off + numel)
            spans.append(SpanSpec(
                [g[sl] for g in self.grads], agg_out=self.agg[sl] if self.write_aggregate else None,
                param=None if self.param is None else self.param[sl],
                fanout=[f[sl] for f in self.fanout],
                bounds=bounds if kind != L.OPT_NONE else (), **self.state_of_span(off, numel)))
        self.span_bucket = [s[3] for s in self.layout.spans]
        self.plan = SyncPlan(spans, kind)
        self._plan_agg = self._plan_opt = self._coef = None
        self._generation = getattr(self, "_generation", 0) + 1     # recorded graphs name the old plan's tables

    # ---- reconfiguration ---------------------------------------------------------
    def reconfigure(self, batches):
        """Changes the set of VSWs (adaptive batching adds or removes workers at run time,
        jabas/train/trainer.py:485-575) without touching weights or optimizer state:
        gradient and replica arenas are added or dropped, the plans rebuilt, the step
        count kept."""
        batches = tuple(batches)
        new_k = len(batches)
        if not 1 <= new_k <= L.MAX_K:
            raise ValueError(f"number of VSWs must be in 1..{L.MAX_K}")
        n = self.layout.total
        in_place = self.in_place
        had_fanout = self._fanout_wanted
        while len(self.grads) < new_k:
            self.grads.append(torch.zeros(n, dtype=self.grad_dtype, device=self.device))
        del self.grads[new_k:]
        if had_fanout and self.param is not None:
            while len(self.fanout) < new_k - 1:
                f = torch.empty(n, dtype=torch.float32, device=self.device)
                f.copy_(self.param)                     # a new replica starts from the main weights
                self.fanout.append(f)
            del self.fanout[max(0, new_k - 1):]
        self.K, self.batches = new_k, batches
        if in_place:
            self.agg = self.grads[0]
        self._build_plan()

    # ---- views -------------------------------------------------------------------
    def _view(self, arena, i):
        off = self.layout.param_offset[i]
        return arena[off:off + self.layout.specs[i].numel]

    def param_view(self, i):
        return self._view(self.param, i)

    def grad_view(self, k, i):
        return self._view(self.grads[k], i)

    def agg_view(self, i):
        return self._view(self.agg, i)

    def bucket_slice(self, b):
        bk = self.layout.buckets[b]
        return slice(bk.offset, bk.offset + bk.numel)

    # ---- the step ----------------------------------------------------------------
    def step_args(self, stats=False, lr_scale=1.0, with_opt=True, accumulations=1):
        opt = self.opt if with_opt else None
        first = self.step_count == 0
        return make_step_args(self.batches, self.grad_dtype, stats=stats, opt=opt, step=self.step_count + 1,
                              first_step=first, lr_scale=lr_scale, accumulations=accumulations)

    def step(self, stats=False, lr_scale=1.0, stream=None, clip_norm=None, accumulations=1):
        """One sync step over the whole gradient set. Returns the per-span stats tensor
        when ``stats`` is set (True / "full": rows of 4 + K sums; "similarity": the four sums of the halves
        and of the aggregate, per-VSW slots zero; "gram", up to eight VSWs: the full row plus the product of
        every pair of VSWs' gradients, ``gram(rows)`` makes the matrix of them).

        Without ``clip_norm``: one fused launch. With it (global-norm clipping as
        examples/gnmt/seq2seq/train/trainer.py:157-161): aggregate + statistics, the
        clipping coefficient on the device, then the optimizer launch over the aggregate
        scaled by it -- the norm has to be known before any weight moves.

        ``accumulations``: micro-batches every VSW summed into its buckets since the last step."""
        out = self._queue(stats, lr_scale, stream, clip_norm, accumulations, None)
        self.step_count += 1
        return out

    def _clipped(self, clip_norm):
        return clip_norm is not None and self.opt is not None

    def _update_args(self, stats, lr_scale, clip_norm, accumulations):
        """Arguments of the launch that moves the weights in the coming step."""
        if not self._clipped(clip_norm):
            return self.step_args(stats=stats, lr_scale=lr_scale, accumulations=accumulations)
        return make_step_args((1,), torch.float32, stats=False, opt=self.opt, step=self.step_count + 1,
                              first_step=self.step_count == 0, lr_scale=lr_scale, grad_scale=self._coef)

    def _queue(self, stats, lr_scale, stream, clip_norm, accumulations, scalars):
        if self._clipped(clip_norm) and self._plan_agg is None:
            self._build_clip_plans()
        args = self._update_args(stats, lr_scale, clip_norm, accumulations)
        if scalars is not None:
            scalars.attach(args)
        if not self._clipped(clip_norm):
            return self.plan.run(args, stream=stream)
        # the norm needs the similarity sums only; a caller that asked for full rows gets them
        level = stats if stats else "similarity"
        rows = self._plan_agg.run(self.step_args(stats=level, with_opt=False, accumulations=accumulations), stream=stream)
        clip_coef(rows, clip_norm, out=self._coef, stream=stream)
        self._plan_opt.run(args, stream=stream)
        return rows if stats else None

    def capture(self, stats=False, clip_norm=None, accumulations=1):
        """Records the step in a HIP graph. The returned object's ``replay(lr_scale=...)`` is ``step`` with
        one graph launch instead of the step's kernel launches; the learning rates, Adam's step count and
        the first-step flag of the moment reach the recorded launch through a block in device memory
        (``StepScalars``) that is refreshed ahead of every replay. Statistics level, clipping and
        ``accumulations`` are fixed by the recording; ``reconfigure`` invalidates it."""
        if self.opt is None:
            raise ValueError("nothing moves between the steps of an engine without optimizer: record its launch directly")
        if self.opt.get("amsgrad", False):
            raise ValueError("the amsgrad kernels take the step's scalars by value only: an amsgrad step cannot be replayed")
        return GraphedStep(self, stats, clip_norm, accumulations)

    def _build_clip_plans(self):
        if self.agg is None:                     # the clipped step passes the aggregate from its first launch to its second
            self.agg = torch.zeros(self.layout.total, dtype=torch.float32, device=self.device)
        agg_spans, opt_spans = [], []
        for (off, numel, bounds, _bucket) in self.layout.spans:
            sl = slice(off, off + numel)
            agg_spans.append(SpanSpec([g[sl] for g in self.grads], agg_out=self.agg[sl]))
            opt_spans.append(SpanSpec([self.agg[sl]], agg_out=self.agg[sl] if self.keep_clipped_grads else None,
                                      param=self.param[sl],
                                      fanout=[f[sl] for f in self.fanout], bounds=bounds,
                                      **self.state_of_span(off, numel)))
        self._plan_agg = SyncPlan(agg_spans, L.OPT_NONE)
        self._plan_opt = SyncPlan(opt_spans, opt_kind(self.opt))
        self._coef = torch.ones(1, dtype=torch.float32, device=self.device)

    def bucket_stats(self, stats):
        """Per-bucket rows from per-span rows (spans of one bucket summed in span order)."""
        rows = stats.detach().cpu()
        out = torch.zeros(len(self.layout.buckets), L.STATS_STRIDE, dtype=torch.float64)
        for i, b in enumerate(self.span_bucket):
            out[b] += rows[i]
        return out

    @staticmethod
    def cosine(stats):
        return cosine_from_stats(stats)

    def gram(self, stats):
        """K x K matrix of the products of the VSWs' gradients over the whole set, from the rows of a step with
        ``stats="gram"`` (float64, on the device)."""
        return gram_from_stats(stats, self.K)


class GraphedStep:
    """A sync step of a ``VSWFlatSync`` recorded once in a HIP graph (``VSWFlatSync.capture``)."""

    def __init__(self, engine, stats, clip_norm, accumulations):
        self.engine, self.stats, self.clip_norm, self.accumulations = engine, stats, clip_norm, accumulations
        self.scalars = StepScalars(engine.device)
        self._generation = engine._generation
        # the first launch out of a code object loads it, which a recording stream must not do: one statistics
        # launch of the same K over a scratch vector first (the per-K kernels, the finalize and coefficient kernels)
        warm = [torch.zeros(4, dtype=engine.grad_dtype, device=engine.device) for _ in range(engine.K)]
        rows = gradient_stats(warm, (1,) * engine.K)
        if engine._clipped(clip_norm):
            if engine._plan_agg is None:
                engine._build_clip_plans()
            clip_coef(gradient_stats([torch.zeros(4, device=engine.device)], (1,)).view(1, -1), 1.0)
        self.scalars.update(engine._update_args(stats, 1.0, clip_norm, accumulations))
        del rows
        torch.cuda.synchronize(engine.device)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.out = engine._queue(stats, 1.0, None, clip_norm, accumulations, self.scalars)

    def replay(self, lr_scale=1.0):
        eng = self.engine
        if eng._generation != self._generation:
            raise RuntimeError("the engine was reconfigured after this step was recorded: record it again")
        self.scalars.update(eng._update_args(self.stats, lr_scale, self.clip_norm, self.accumulations))
        self.graph.replay()
        eng.step_count += 1
        return self.out
