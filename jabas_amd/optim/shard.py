"""ShardSGD / ShardAdam / ShardAdamW: optimizers whose ``step(gradients)`` updates only the
parameters a DDP bucket carries, for the "overlap" weight-sync mode.

Stand in for ``iidp.optim`` (un-vendored IIDP submodule). The surface is taken from the
call sites (examples/resnet50/main.py:351-355, examples/vit/main.py:434-435,
examples/faster_r_cnn/train.py:269-272) and from the one vendored subclass,
examples/gnmt/seq2seq/train/shard_optimizer.py:8-90: constructor arguments of the torch
optimizer of the same name, ``step(gradients)`` with gradients matched to parameters by
their ``.index`` attribute, lazy state, torch 1.8.1 formulas. ``step()`` without
arguments updates every parameter from its ``.grad`` (the "sequential" mode).

Every update is one fused launch over a table of (gradient, weight, state) spans through
the C ABI instead of 4 (SGD) or ~10 (Adam) elementwise kernels per tensor.
"""
import torch

from .. import _lib as L
from .. import sync


def _index_of(t):
    idx = getattr(t, "index", None)       # the attribute the reference sets; anything callable is not it
    return idx if isinstance(idx, int) else None


class _ShardOptimizer(torch.optim.Optimizer):
    _kind = None
    _max_cached_plans = 1024       # one per distinct call (a DDP bucket each in the overlap mode): a few KB of tables apiece

    def __init__(self, params, defaults):
        super().__init__(params, defaults)
        self._plans = {}
        self._recipes = {}          # call signature -> prepared launches (see _signature)
        self._replicas = {}         # id(parameter) -> the same parameter of the other VSW replicas

    def attach_replicas(self, main_params=(), *replica_params):
        """``main_params``: the parameters of the model this optimizer updates; ``replica_params``: those of the
        other VSW replicas on this GPU, one iterable per replica, in the same order (``model.parameters()`` of
        identically built models). Every update then also writes the new weights into the replicas, in the
        same launch (4 more bytes written per element and replica, nothing read again), which is the copy of
        the main VSW's weights to the other VSWs that follows the optimizer step in IIDP
        (jabas/train/trainer.py:530-534 shows the same copy when VSWs are added). Call again after replacing a
        replica's tensors; call without arguments to detach."""
        mine = list(main_params)
        held = {id(p) for group in self.param_groups for p in group["params"]}
        if len(replica_params) > L.MAX_K - 1:
            raise ValueError(f"at most {L.MAX_K - 1} replicas")
        if replica_params and not held <= {id(p) for p in mine}:
            raise ValueError("main_params must hold every parameter of the optimizer")
        table = {}
        for r, params in enumerate(replica_params):
            theirs = list(params)
            if len(theirs) != len(mine):
                raise ValueError(f"replica {r} has {len(theirs)} parameters, the main model {len(mine)}")
            for p, q in zip(mine, theirs):
                if id(p) not in held:
                    continue
                if q is p or q.shape != p.shape or q.dtype != torch.float32 or q.device != p.device:
                    raise ValueError(f"replica {r}: a parameter does not mirror the main model's (shape, dtype, "
                                     "device, or it is the very same tensor)")
                if not q.is_contiguous():
                    raise ValueError(f"replica {r}: parameters must be contiguous")
                table.setdefault(id(p), []).append(q)
        self._replicas = table
        self._plans.clear()
        self._recipes.clear()
        return self

    def _fanout(self, p):
        """Flat views of p's replicas for the launch; a replica that sits at another position of a 16-byte line
        than p cannot share p's vector accesses and is copied after the launch instead."""
        views = []
        for q in self._replicas.get(id(p), ()):
            if self._congruent(q.data, p):
                views.append(q.data.view(-1))
            else:
                self._late_copies.append((q, p))
        return views

    def load_state_dict(self, state_dict):
        super().load_state_dict(state_dict)
        self._plans.clear()         # the state tensors were replaced: prepared launches point at the old ones
        self._recipes.clear()

    # -- prepared calls -----------------------------------------------------------------
    # A training loop hands step() the same parameters and the same gradient buffers every iteration
    # (DDP bucket views keep their addresses). Matching, validating and marshalling ~150 tensors costs
    # more host time than the launch takes on the GPU, so a call that found every state in place is
    # remembered under its signature, and repeated calls only refresh the launch scalars.
    def _signature(self, pairs):
        rep = self._replicas
        if not rep:
            return tuple([(p.data_ptr(), g.data_ptr(), g.numel()) for _, p, g in pairs])
        return tuple([(p.data_ptr(), g.data_ptr(), g.numel()) + tuple(q.data_ptr() for q in rep.get(id(p), ()))
                      for _, p, g in pairs])

    def _remember(self, sig, launches, copies):
        if len(self._recipes) >= self._max_cached_plans:
            self._recipes.clear()
        self._recipes[sig] = (launches, copies, list(self._late_copies))

    _late_copies = ()

    def _copy_late(self, late):
        for q, p in late:
            q.data.copy_(p.data)

    # -- matching ---------------------------------------------------------------------
    def _pairs(self, gradients):
        """[(group_index, param, grad)] for this call."""
        out = []
        if gradients is None:
            for gi, group in enumerate(self.param_groups):
                for p in group["params"]:
                    if p.grad is not None:
                        out.append((gi, p, p.grad))
            return out
        by_index = {}
        for g in gradients:
            idx = _index_of(g)
            if idx is None:
                raise ValueError("step(gradients): every gradient needs an .index attribute naming its parameter")
            by_index[idx] = g
        for gi, group in enumerate(self.param_groups):
            for p in group["params"]:
                g = by_index.get(_index_of(p))
                if g is not None and _index_of(p) is not None:
                    out.append((gi, p, g))
        return out

    @staticmethod
    def _congruent(g, p):
        return (g.data_ptr() // 4) % 4 == (p.data_ptr() // 4) % 4

    def _prepare(self, p, g):
        if g.is_sparse:
            raise RuntimeError(f"{type(self).__name__} does not support sparse gradients")
        if not p.is_cuda:
            raise RuntimeError(f"{type(self).__name__} updates GPU parameters only (no CPU fallback)")
        if g.dtype != torch.float32 or p.dtype != torch.float32:
            raise TypeError("fp32 parameters and gradients expected")
        g = g.detach()
        if not g.is_contiguous():
            g = g.contiguous()
            self._volatile = True                 # a fresh copy every call: nothing to remember
        g = g.view(-1)
        if not self._congruent(g, p):
            # a bucket view that starts off the weight's position in a 16-byte line: realign a copy
            skew = (p.data_ptr() // 4) % 4
            buf = torch.empty(g.numel() + 4, dtype=torch.float32, device=g.device)
            base = (buf.data_ptr() // 4) % 4
            tmp = buf[(skew - base) % 4:][:g.numel()]
            tmp.copy_(g)
            self._copies.append((tmp, g))
            g = tmp
        return g

    def _launch(self, spans, args):
        key = (args.opt_kind,) + tuple((s.grads[0].data_ptr(), s.param.data_ptr(), s.grads[0].numel(), s.bounds[0][1],
                                         s.agg_out is not None) + tuple(f.data_ptr() for f in s.fanout) for s in spans)
        plan = self._plans.get(key)
        if plan is None:
            if len(self._plans) >= self._max_cached_plans:
                self._plans.clear()
            plan = self._plans[key] = sync.SyncPlan(spans, args.opt_kind)
        plan.run(args)
        return plan

    def _new_args(self, kind):
        a = L.JabasStepArgs()
        a.K = 1
        a.grad_dtype = L.F32
        a.weight[0] = 1.0                       # g * 1.0f is exact: the gradient goes in unchanged
        a.half_weight[0] = 1.0
        a.opt_kind = kind
        scale = getattr(self, "_grad_scale", None)
        if scale is not None:                   # device scalar of a clipped step
            a.grad_scale = scale.data_ptr()
        return a


class ShardSGD(_ShardOptimizer):
    def __init__(self, params, lr, momentum=0, dampening=0, weight_decay=0, nesterov=False):
        if lr < 0.0:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if momentum < 0.0:
            raise ValueError("Invalid momentum value: {}".format(momentum))
        if weight_decay < 0.0:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        if nesterov and (momentum <= 0 or dampening != 0):
            raise ValueError("Nesterov momentum requires a momentum and zero dampening")
        super().__init__(params, dict(lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                                      nesterov=nesterov))

    @torch.no_grad()
    def step(self, gradients=None, closure=None):
        loss = closure() if closure is not None else None
        pairs = self._pairs(gradients)
        sig = self._signature(pairs)
        if self._replay(self._recipes.get(sig)):
            return loss
        self._copies, self._volatile, launches, self._late_copies = [], False, [], []
        # launches are split by (momentum, dampening, nesterov, first-step): launch-wide scalars
        batches = {}
        for gi, p, g in pairs:
            group = self.param_groups[gi]
            st = self.state[p]
            first = group["momentum"] != 0 and "momentum_buffer" not in st
            if first:
                st["momentum_buffer"] = torch.empty_like(p, memory_format=torch.preserve_format)
            key = (group["momentum"], group["dampening"], bool(group["nesterov"]), first)
            batches.setdefault(key, []).append((gi, p, self._prepare(p, g), st.get("momentum_buffer")))
        for (momentum, dampening, nesterov, first), items in batches.items():
            slots, spans = {}, []
            args = self._new_args(L.OPT_SGD)
            for gi, p, g, buf in items:
                slot = slots.setdefault(gi, len(slots))
                if slot >= L.MAX_GROUPS:
                    raise RuntimeError(f"more than {L.MAX_GROUPS} parameter groups in one launch")
                spans.append(sync.SpanSpec([g], param=p.data.view(-1), state1=None if buf is None else buf.view(-1),
                                           fanout=self._fanout(p), bounds=((0, slot),)))
            for gi, slot in slots.items():
                args.groups[slot].lr = float(self.param_groups[gi]["lr"])
                args.groups[slot].weight_decay = float(self.param_groups[gi]["weight_decay"])
                args.groups[slot].step = 1
            args.n_groups = len(slots)
            args.momentum, args.dampening = float(momentum), float(dampening)
            args.nesterov, args.first_step = int(nesterov), int(first)
            plan = self._launch(spans, args)
            launches.append((plan, args, (momentum, dampening, bool(nesterov)), list(slots.items())))
            self._volatile = self._volatile or first
        self._copy_late(self._late_copies)
        if not self._volatile:
            self._remember(sig, launches, self._copies)
        return loss

    def _replay(self, recipe):
        """Repeats a remembered call with the hyperparameters as the groups hold them now. False (and
        nothing done) when a group changed a scalar the launches were split by."""
        if recipe is None:
            return False
        launches, copies, late = recipe
        for _, _, key, slots in launches:
            for gi, _ in slots:
                group = self.param_groups[gi]
                if (group["momentum"], group["dampening"], bool(group["nesterov"])) != key:
                    return False
        for tmp, g in copies:
            tmp.copy_(g)
        for plan, args, _, slots in launches:
            for gi, slot in slots:
                args.groups[slot].lr = float(self.param_groups[gi]["lr"])
                args.groups[slot].weight_decay = float(self.param_groups[gi]["weight_decay"])
            plan.run(args)
        self._copy_late(late)
        return True


class ShardAdam(_ShardOptimizer):
    _adamw = False

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False):
        if not 0.0 <= lr:
            raise ValueError("Invalid learning rate: {}".format(lr))
        if not 0.0 <= eps:
            raise ValueError("Invalid epsilon value: {}".format(eps))
        if not 0.0 <= betas[0] < 1.0:
            raise ValueError("Invalid beta parameter at index 0: {}".format(betas[0]))
        if not 0.0 <= betas[1] < 1.0:
            raise ValueError("Invalid beta parameter at index 1: {}".format(betas[1]))
        if not 0.0 <= weight_decay:
            raise ValueError("Invalid weight_decay value: {}".format(weight_decay))
        super().__init__(params, dict(lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad))

    @torch.no_grad()
    def step(self, gradients=None, closure=None):
        loss = closure() if closure is not None else None
        pairs = self._pairs(gradients)
        sig = self._signature(pairs)
        if self._replay(self._recipes.get(sig)):
            return loss
        self._copies, self._volatile, launches, self._late_copies = [], False, [], []
        batches = {}
        write_back = getattr(self, "_grad_scale", None) is not None     # a clipped step leaves the clipped gradients behind
        for gi, p, g in pairs:
            group = self.param_groups[gi]
            amsgrad = bool(group["amsgrad"])
            st = self.state[p]
            if len(st) == 0:
                self._volatile = True             # state created in this call: remember the next one
                st["step"] = 0
                st["exp_avg"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                st["exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
                if amsgrad:                       # the maximum of the second moment so far (shard_optimizer.py:58-60)
                    st["max_exp_avg_sq"] = torch.zeros_like(p, memory_format=torch.preserve_format)
            elif amsgrad and "max_exp_avg_sq" not in st:
                raise RuntimeError("amsgrad was switched on after the state was created: no max_exp_avg_sq to continue from")
            st["step"] += 1
            key = (tuple(group["betas"]), group["eps"], amsgrad)
            batches.setdefault(key, []).append((gi, int(st["step"]), p, self._prepare(p, g), st))
        for (betas, eps, amsgrad), items in batches.items():
            slots, spans = {}, []
            if amsgrad:
                args = self._new_args(L.OPT_ADAMW_AMSGRAD if self._adamw else L.OPT_ADAM_AMSGRAD)
            else:
                args = self._new_args(L.OPT_ADAMW if self._adamw else L.OPT_ADAM)
            for gi, step, p, g, st in items:
                slot = slots.setdefault((gi, step), len(slots))
                if slot >= L.MAX_GROUPS:
                    raise RuntimeError(f"more than {L.MAX_GROUPS} (group, step) combinations in one launch")
                spans.append(sync.SpanSpec([g], agg_out=g if write_back else None, param=p.data.view(-1),
                                           state1=st["exp_avg"].view(-1), state2=st["exp_avg_sq"].view(-1),
                                           state3=st["max_exp_avg_sq"].view(-1) if amsgrad else None,
                                           fanout=self._fanout(p), bounds=((0, slot),)))
            for (gi, step), slot in slots.items():
                args.groups[slot].lr = float(self.param_groups[gi]["lr"])
                args.groups[slot].weight_decay = float(self.param_groups[gi]["weight_decay"])
                args.groups[slot].step = step
            args.n_groups = len(slots)
            args.beta1, args.beta2, args.eps = float(betas[0]), float(betas[1]), float(eps)
            plan = self._launch(spans, args)
            # per slot: its group and one state that carries the slot's step count; per item: state and slot
            reps = {}
            for gi, step, p, g, st in items:
                reps.setdefault(slots[(gi, step)], (gi, st))
            launches.append((plan, args, (betas, eps, amsgrad), sorted(reps.items()),
                             [(st, slots[(gi, step)]) for gi, step, p, g, st in items]))
        if write_back:
            for tmp, g in self._copies:           # gradients that were realigned into a copy: the clipped values go back
                g.copy_(tmp)
        self._copy_late(self._late_copies)
        if not self._volatile:
            self._remember(sig, launches, self._copies)
        return loss

    def _replay(self, recipe):
        """Repeats a remembered call: bumps every parameter's step count and refreshes the launch scalars.
        False (and nothing done) when betas / eps of a group changed or when parameters that shared a
        step count no longer do (they were stepped apart in between)."""
        if recipe is None:
            return False
        launches, copies, late = recipe
        for _, _, key, reps, items in launches:
            for _, (gi, _) in reps:
                group = self.param_groups[gi]
                if (tuple(group["betas"]), group["eps"], bool(group["amsgrad"])) != key:
                    return False
            steps = [st["step"] for _, (_, st) in reps]
            for st, slot in items:
                if st["step"] != steps[slot]:
                    return False
        for tmp, g in copies:
            tmp.copy_(g)
        for plan, args, _, reps, items in launches:
            for st, _ in items:
                st["step"] += 1
            for slot, (gi, st) in reps:
                args.groups[slot].lr = float(self.param_groups[gi]["lr"])
                args.groups[slot].weight_decay = float(self.param_groups[gi]["weight_decay"])
                args.groups[slot].step = int(st["step"])
            plan.run(args)
        if getattr(self, "_grad_scale", None) is not None:
            for tmp, g in copies:
                g.copy_(tmp)
        self._copy_late(late)
        return True


class ShardAdamW(ShardAdam):
    _adamw = True

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=1e-2, amsgrad=False):
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)


class ShardGNMTAdam(ShardAdam):
    """ShardAdam with gradient clipping inside ``step`` (examples/gnmt/seq2seq/train/shard_optimizer.py:8-90):
    the gradients handed to one ``step(gradients)`` call (one DDP bucket in the overlap mode) are scaled to a
    joint 2-norm of at most ``grad_clip`` before the update, torch.nn.utils.clip_grad_norm_'s rule
    (coefficient max_norm / (norm + 1e-6), applied when below 1). One statistics launch over the gradients
    forms the norm, the coefficient stays on the device, and the Adam launch multiplies it in and writes the
    scaled gradients back in place, as ``clip_grad_norm_for_overlap`` leaves the tensors it was handed
    (shard_optimizer.py:75-76): a caller that reads gradient norms after the step sees the clipped ones."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0, amsgrad=False,
                 grad_clip=float('inf')):
        super().__init__(params, lr=lr, betas=betas, eps=eps, weight_decay=weight_decay, amsgrad=amsgrad)
        self.grad_clip = grad_clip
        self._clip_plans = {}
        self._coef = None
        if len(self.param_groups) > 1:
            raise ValueError(
                "Length of self.param_groups must not be > 1 "
                "because of applying gradient clipping")

    @torch.no_grad()
    def step(self, gradients=None, closure=None):
        if self.grad_clip == float('inf'):
            return super().step(gradients, closure)
        pairs = self._pairs(gradients)
        if not pairs:
            return super().step(gradients, closure)
        flat = []
        for _, p, g in pairs:
            if g.is_sparse:
                raise RuntimeError('Adam does not support sparse gradients, please consider SparseAdam instead')
            if not p.is_cuda:
                raise RuntimeError(f"{type(self).__name__} updates GPU parameters only (no CPU fallback)")
            g = g.detach()
            flat.append((g if g.is_contiguous() else g.contiguous()).view(-1))
        sig = tuple((g.data_ptr(), g.numel()) for g in flat)
        plan = self._clip_plans.get(sig)
        if plan is None:
            if len(self._clip_plans) >= self._max_cached_plans:
                self._clip_plans.clear()
            plan = self._clip_plans[sig] = sync.SyncPlan([sync.SpanSpec([g]) for g in flat], L.OPT_NONE)
        args = L.JabasStepArgs()
        args.K, args.grad_dtype, args.stats, args.opt_kind = 1, L.F32, 1, L.OPT_NONE
        args.weight[0] = args.half_weight[0] = 1.0
        rows = plan.run(args)
        if self._coef is None:
            self._coef = torch.ones(1, dtype=torch.float32, device=flat[0].device)
        sync.clip_coef(rows, self.grad_clip, out=self._coef)
        self._grad_scale = self._coef
        try:
            return super().step(gradients, closure)
        finally:
            self._grad_scale = None
