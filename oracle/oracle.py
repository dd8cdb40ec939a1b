"""CPU oracle of the per-GPU gradient-sync path. TEST INFRASTRUCTURE, not product code:
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

It restates, with plain torch CPU ops, what the reference computes for this path. Every
fp32 product and sum is a separate torch op (``torch.mul`` then ``torch.add`` without
``alpha=``), so each is rounded on its own and the order of operations is the one
written here; ATen's ``add(alpha=)`` is avoided because its vectorised body fuses the
multiply-add while its scalar tail does not.

Reference files followed (JABAS repository):
  aggregate        jabas/train/trainer.py:452-468,594-599 (only VSW 0 communicates; per-GPU
                   batch = LBS x K), jabas/ddp_comm_hooks/similarity_allreduce.py:32
                   (sum, then division by the worker count)
  statistics       jabas/ddp_comm_hooks/similarity_allreduce.py:20-35 (half-group mean
                   gradient per bucket), jabas/train/trainer.py:427-432 (parity split),
                   :470-483 (cat over buckets + cosine_similarity)
  SGD              torch 1.8.1 optim/_functional.sgd, called through
                   examples/resnet50/main.py:351-359, examples/faster_r_cnn/train.py:266-276
  Adam / AdamW     torch 1.8.1 optim/_functional.adam / adamw, called through
                   examples/gnmt/seq2seq/train/shard_optimizer.py:78-90, examples/vit/main.py:425-437

Pinning. The arithmetic of IIDP's local aggregation and of Shard*.step lives in the
un-vendored ``iidp`` submodule and a patched torch 1.8.1, neither present: the order of
the aggregate (a1), the place of the division, and Shard* == torch 1.8.1 _functional are
assumptions of this file -> PARITY UNPINNED against the reference for those. What is
pinned, in tests/test_oracle_*.py: every function against an independent C restatement
(oracle/oracle_c.c, bit for bit), against scalar numpy.float32 brute force, against
torch.optim.SGD/Adam/AdamW and torch.nn.functional.cosine_similarity / torch.dot in
float64 as library routines, and against closed forms and invariants.
"""
import math

import numpy as np
import torch

STATS_STRIDE = 20          # the four sums and up to 16 per-worker norms (the library's rows are wider: pair products too)
DOT_AB, NORM_A, NORM_B, NORM_AGG, NORM_VSW0 = 0, 1, 2, 3, 4


# ------------------------------------------------------------------------------ weights
def batch_weights(batches, half_id=None, accumulations=1):
    """w_k = fp32(b_k / (B * accumulations)) with the quotient formed in double; half weights likewise
    over each half's own batch total. Default halves: even VSW index -> A, odd -> B. accumulations =
    micro-batches summed into each bucket before the step (every one of them a decoupled worker in the
    reference's count, jabas/train/trainer.py:594-599)."""
    b = [float(x) for x in batches]
    K = len(b)
    total = math.fsum(b) * float(int(accumulations))
    w = [float(np.float32(x / total)) for x in b]
    if half_id is None:
        half_id = [k % 2 for k in range(K)]
    acc = float(int(accumulations))
    tot = [math.fsum(x for x, h in zip(b, half_id) if h == 0) * acc, math.fsum(x for x, h in zip(b, half_id) if h == 1) * acc]
    hw = [float(np.float32(b[k] / tot[half_id[k]])) for k in range(K)]
    return w, list(half_id), hw


def _f32(t):
    return t.detach().to("cpu").to(torch.float32)     # bf16 -> fp32 widening is exact


def _weighted_sum(grads, ws):
    """acc = g_0*w_0; acc = acc + g_k*w_k, each op rounded to fp32."""
    acc = None
    for g, w in zip(grads, ws):
        t = torch.mul(_f32(g), w)
        acc = t if acc is None else torch.add(acc, t)
    return acc


# ---------------------------------------------------------------------------- aggregate
def aggregate(grads, batches):
    w, _, _ = batch_weights(batches)
    return _weighted_sum(grads, w)


def half_aggregates(grads, batches, half_id=None):
    _, hid, hw = batch_weights(batches, half_id)
    n = grads[0].numel()
    out = []
    for h in (0, 1):
        sel = [(g, w) for g, w, i in zip(grads, hw, hid) if i == h]
        out.append(_weighted_sum([g for g, _ in sel], [w for _, w in sel]) if sel
                   else torch.zeros(n, dtype=torch.float32))
    return out


# --------------------------------------------------------------------------- statistics
def stats(grads, batches, half_id=None):
    """Statistics row of one span: float64 tensor of STATS_STRIDE entries."""
    K = len(grads)
    ga, gb = half_aggregates(grads, batches, half_id)
    agg = aggregate(grads, batches)
    row = torch.zeros(STATS_STRIDE, dtype=torch.float64)
    da, db, dg = ga.double(), gb.double(), agg.double()
    row[DOT_AB] = torch.dot(da, db)
    row[NORM_A] = torch.dot(da, da)
    row[NORM_B] = torch.dot(db, db)
    row[NORM_AGG] = torch.dot(dg, dg)
    for k in range(K):
        d = _f32(grads[k]).double()
        row[NORM_VSW0 + k] = torch.dot(d, d)
    return row


def gram(grads):
    d = torch.stack([_f32(g).double() for g in grads])
    return d @ d.t()


def cosine(dot, na, nb, eps=1e-8):
    """torch 1.8.1 cosine_similarity: dot / sqrt(max(|a|^2 |b|^2, eps^2))."""
    return dot / math.sqrt(max(na * nb, eps * eps))


def cosine_from_rows(rows, eps=1e-8):
    rows = rows.reshape(-1, STATS_STRIDE).double()
    return cosine(float(rows[:, DOT_AB].sum()), float(rows[:, NORM_A].sum()), float(rows[:, NORM_B].sum()), eps)


# ---------------------------------------------------------------------------- optimizer
def sgd_step(p, g, buf, lr, weight_decay=0.0, momentum=0.0, dampening=0.0, nesterov=False, first_step=False):
    """torch 1.8.1 _functional.sgd on one tensor, in place on p (and buf)."""
    d = g
    if weight_decay != 0:
        d = torch.add(d, torch.mul(p, weight_decay))
    if momentum != 0:
        if first_step:
            buf.copy_(d)
        else:
            buf.copy_(torch.add(torch.mul(buf, momentum), torch.mul(d, 1 - dampening)))
        d = torch.add(d, torch.mul(buf, momentum)) if nesterov else buf
    p.copy_(torch.add(p, torch.mul(d, -lr)))


def _ieee_sqrt(t):
    """Correctly rounded fp32 square root (what sqrtf is on the GPUs the reference runs on).
    torch.sqrt on CPU goes through MKL's vector maths for large contiguous tensors and is
    off by one ulp for about 0.6 % of inputs; numpy's sqrt is the hardware instruction."""
    return torch.from_numpy(np.sqrt(t.detach().contiguous().numpy()))


def adam_step(p, g, m, v, lr, weight_decay, betas, eps, step, adamw, vmax=None):
    """torch 1.8.1 _functional.adam / adamw on one tensor, in place. ``vmax``: the running maximum of the
    second moment (``max_exp_avg_sq``) when amsgrad is on, as ShardGNMTAdam.step threads it into F.adam
    (examples/gnmt/seq2seq/train/shard_optimizer.py:58-66,79-90): torch.maximum(max_exp_avg_sq, exp_avg_sq,
    out=max_exp_avg_sq), and the denominator is formed from the maximum."""
    beta1, beta2 = betas
    bc1 = 1 - beta1 ** step
    bc2 = 1 - beta2 ** step
    if adamw:
        p.copy_(torch.mul(p, 1 - lr * weight_decay))
    elif weight_decay != 0:
        g = torch.add(g, torch.mul(p, weight_decay))
    m.copy_(torch.add(torch.mul(m, beta1), torch.mul(g, 1 - beta1)))
    v.copy_(torch.add(torch.mul(v, beta2), torch.mul(torch.mul(g, 1 - beta2), g)))
    if vmax is not None:
        vmax.copy_(torch.maximum(vmax, v))
    denom = torch.add(torch.div(_ieee_sqrt(v if vmax is None else vmax), math.sqrt(bc2)), eps)
    step_size = lr / bc1
    p.copy_(torch.add(p, torch.div(torch.mul(m, -step_size), denom)))


def opt_step(opt, group, p, g, s1, s2, step, first_step, lr_scale=1.0, s3=None):
    """Dispatch on the optimizer dictionary used throughout the build (``s3``: max_exp_avg_sq when
    ``opt['amsgrad']``)."""
    grp = opt["groups"][group]
    lr = grp["lr"] * lr_scale
    step = grp.get("step", step)               # a group may carry its own Adam step count
    wd = grp.get("weight_decay", 0.0)
    if opt["kind"] == "sgd":
        sgd_step(p, g, s1, lr, wd, opt.get("momentum", 0.0), opt.get("dampening", 0.0),
                 opt.get("nesterov", False), first_step)
    elif opt["kind"] in ("adam", "adamw"):
        if bool(opt.get("amsgrad", False)) != (s3 is not None):
            raise ValueError("amsgrad needs the max_exp_avg_sq tensor, and only amsgrad takes one")
        adam_step(p, g, s1, s2, lr, wd, opt.get("betas", (0.9, 0.999)), opt.get("eps", 1e-8), step,
                  opt["kind"] == "adamw", vmax=s3)
    else:
        raise ValueError(opt["kind"])


# -------------------------------------------------------------------------- clipping
def clip_coef(total_sq, max_norm, eps=1e-6):
    """torch.nn.utils.clip_grad_norm_: clip_coef = max_norm / (total_norm + 1e-6), applied
    only when below 1 (examples/gnmt/seq2seq/train/trainer.py:157-161). The norm is formed
    from the float64 sum of squares; the coefficient is an fp32 scalar."""
    return float(np.float32(max_norm / (math.sqrt(total_sq) + eps)))


def clip(agg, max_norm, eps=1e-6):
    """Returns (clipped aggregate, coefficient); one fp32 product per element when clipping."""
    c = clip_coef(float(torch.dot(agg.double(), agg.double())), max_norm, eps)
    return (torch.mul(agg, c) if c < 1.0 else agg), c


# ---------------------------------------------------------------------- whole sync step
def sync_step(grads, batches, spans, opt=None, param=None, state1=None, state2=None, step=1, first_step=False,
              want_stats=False, half_id=None, lr_scale=1.0, clip_norm=None, state3=None):
    """Fused-step semantics over flat CPU arenas.

    grads: K flat tensors; spans: [(offset, numel, bounds)] with bounds [(start, group)].
    Returns (aggregate arena fp32, stats rows or None); updates param/state in place.
    """
    agg = torch.zeros(grads[0].numel(), dtype=torch.float32)
    rows = torch.zeros(len(spans), STATS_STRIDE, dtype=torch.float64) if want_stats else None
    for si, (off, n, bounds) in enumerate(spans):
        sl = slice(off, off + n)
        gs = [g[sl] for g in grads]
        agg[sl] = aggregate(gs, batches)
        if want_stats:
            rows[si] = stats(gs, batches, half_id)
    if clip_norm is not None:                  # global norm over every span, then one scale
        total = sum(float(torch.dot(agg[o:o + n].double(), agg[o:o + n].double())) for o, n, _ in spans)
        c = clip_coef(total, clip_norm)
        if c < 1.0:
            for o, n, _ in spans:
                agg[o:o + n] = torch.mul(agg[o:o + n], c)
    for si, (off, n, bounds) in enumerate(spans):
        if opt is not None:
            bl = list(bounds) if bounds else [(0, 0)]
            for j, (start, group) in enumerate(bl):
                end = bl[j + 1][0] if j + 1 < len(bl) else n
                s2_ = slice(off + start, off + end)
                opt_step(opt, group, param[s2_], agg[s2_],
                         None if state1 is None else state1[s2_],
                         None if state2 is None else state2[s2_], step, first_step, lr_scale,
                         None if state3 is None else state3[s2_])
    return agg, rows
