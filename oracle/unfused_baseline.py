"""The reference's unfused launch structure for one sync step, on the CPU, for timing.
TEST INFRASTRUCTURE: only bench.py's cpu_baseline leg and tests/ may import it.

The reference's own Python cannot run here (it needs the un-vendored ``iidp`` package
and a patched torch 1.8.1), so this restates its structure with stock torch CPU ops:

  * local aggregation of the K VSW buckets into VSW 0's bucket, one in-place pass per
    worker (jabas/train/trainer.py:452-468: only VSW 0 communicates; the others hand
    their buckets over);
  * on statistic steps, per bucket, a clone + scale per half
    (jabas/ddp_comm_hooks/similarity_allreduce.py:27-32), then ``torch.cat`` over all
    buckets and ``cosine_similarity(a, b, dim=0)`` (jabas/train/trainer.py:470-483);
  * the single-tensor optimizer loop of torch.optim.SGD / Adam / AdamW with one
    Parameter per model tensor and the reference's parameter groups
    (examples/resnet50/main.py:340-359, examples/vit/main.py:405-437).
"""
import torch

from . import oracle as O


class UnfusedStep:
    def __init__(self, layout, batches, grad_dtype, grad_std, opt, seed=0):
        self.layout, self.batches, self.opt = layout, tuple(batches), opt
        self.K = len(batches)
        n = layout.total
        gen = torch.Generator().manual_seed(seed)
        self.grads = [(torch.randn(n, generator=gen) * grad_std).to(grad_dtype) for _ in range(self.K)]
        self.main = self.grads[0] if grad_dtype == torch.float32 else torch.zeros(n, dtype=torch.float32)
        self.param = torch.randn(n, generator=gen) * 0.05
        self.params = []
        groups = [dict(params=[], **{k: v for k, v in g.items()}) for g in opt["groups"]]
        for i, spec in enumerate(layout.specs):
            off = layout.param_offset[i]
            p = torch.nn.Parameter(self.param[off:off + spec.numel])
            p.grad = self.main[off:off + spec.numel]
            groups[spec.group]["params"].append(p)
            self.params.append(p)
        groups = [g for g in groups if g["params"]]
        if opt["kind"] == "sgd":
            self.optim = torch.optim.SGD(groups, lr=groups[0]["lr"], momentum=opt.get("momentum", 0.0),
                                         dampening=opt.get("dampening", 0.0), nesterov=opt.get("nesterov", False),
                                         foreach=False)
        else:
            cls = torch.optim.AdamW if opt["kind"] == "adamw" else torch.optim.Adam
            self.optim = cls(groups, lr=groups[0]["lr"], betas=opt.get("betas", (0.9, 0.999)),
                             eps=opt.get("eps", 1e-8), foreach=False)
        self.w, self.hid, self.hw = O.batch_weights(self.batches)

    @torch.no_grad()
    def step(self, want_stats):
        cos = None
        if want_stats:
            halves = ([], [])
            for b in self.layout.buckets:
                sl = slice(b.offset, b.offset + b.numel)
                for h in (0, 1):
                    acc = None
                    for g, wk, i in zip(self.grads, self.hw, self.hid):
                        if i != h:
                            continue
                        t = g[sl].detach().clone().float().mul_(wk) if g.dtype != torch.float32 \
                            else g[sl].detach().clone().mul_(wk)
                        acc = t if acc is None else acc.add_(t)
                    halves[h].append(acc if acc is not None else torch.zeros(b.numel))
            a, b_ = torch.cat(halves[0]), torch.cat(halves[1])
            cos = float(torch.nn.functional.cosine_similarity(a, b_, dim=0))
        if self.main is self.grads[0]:
            self.main.mul_(self.w[0])
        else:
            torch.mul(self.grads[0].float(), self.w[0], out=self.main)
        for g, wk in zip(self.grads[1:], self.w[1:]):
            self.main.add_(g if g.dtype == torch.float32 else g.float(), alpha=wk)
        self.optim.step()
        return cos
