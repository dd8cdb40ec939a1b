"""ctypes front of oracle/oracle_c.c (scalar C restatement). TEST INFRASTRUCTURE: only
tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import it.

Takes and returns torch CPU tensors; the fp32 scalars handed to C are derived here from
Python doubles (``1 - beta1 ** step`` etc.) exactly as torch 1.8.1's Python optimizer
code derives them before they reach an fp32 kernel.
"""
import ctypes as C
import math
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle_c.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "liboracle_c.so"], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
    return _lib


def _f(x):
    return C.c_float(float(np.float32(x)))


def _grad_ptrs(grads):
    bf16 = grads[0].dtype == torch.bfloat16
    keep = [g.detach().cpu().contiguous() for g in grads]
    arr = (C.c_void_p * len(keep))(*[g.data_ptr() for g in keep])
    return arr, int(bf16), keep


def aggregate(grads, w):
    arr, bf16, keep = _grad_ptrs(grads)
    n = keep[0].numel()
    out = torch.empty(n, dtype=torch.float32)
    cw = (C.c_float * len(w))(*[float(x) for x in w])
    lib().oc_aggregate(arr, len(keep), bf16, cw, C.c_void_p(out.data_ptr()), C.c_size_t(n))
    return out


def stats(grads, w, half_id, hw):
    arr, bf16, keep = _grad_ptrs(grads)
    n, K = keep[0].numel(), len(keep)
    row = torch.zeros(20, dtype=torch.float64)          # 4 + 16 slots: the oracle's own rows (four sums, one norm per worker)
    lib().oc_stats(arr, K, bf16, (C.c_float * K)(*[float(x) for x in w]), (C.c_uint8 * K)(*[int(x) for x in half_id]),
                   (C.c_float * K)(*[float(x) for x in hw]), C.c_size_t(n), C.c_void_p(row.data_ptr()))
    return row


def gram(grads):
    arr, bf16, keep = _grad_ptrs(grads)
    n, K = keep[0].numel(), len(keep)
    out = torch.zeros(K, K, dtype=torch.float64)
    lib().oc_gram(arr, K, bf16, C.c_size_t(n), C.c_void_p(out.data_ptr()))
    return out


def sgd_step(p, g, buf, lr, weight_decay=0.0, momentum=0.0, dampening=0.0, nesterov=False, first_step=False):
    n = p.numel()
    lib().oc_sgd(C.c_void_p(p.data_ptr()), C.c_void_p(g.data_ptr()), C.c_void_p(buf.data_ptr() if buf is not None else 0),
                 C.c_size_t(n), _f(weight_decay), _f(-lr), _f(momentum), _f(1 - dampening),
                 int(momentum != 0), int(first_step), int(nesterov))


def adam_step(p, g, m, v, lr, weight_decay, betas, eps, step, adamw, vmax=None):
    beta1, beta2 = betas
    bc1 = 1 - beta1 ** step
    bc2 = 1 - beta2 ** step
    lib().oc_adam(C.c_void_p(p.data_ptr()), C.c_void_p(g.data_ptr()), C.c_void_p(m.data_ptr()), C.c_void_p(v.data_ptr()),
                  C.c_void_p(vmax.data_ptr() if vmax is not None else 0), C.c_size_t(p.numel()), _f(weight_decay), _f(1 - lr * weight_decay), _f(beta1), _f(1 - beta1),
                  _f(beta2), _f(1 - beta2), _f(math.sqrt(bc2)), _f(eps), _f(-(lr / bc1)), int(adamw))
