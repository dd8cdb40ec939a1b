"""CPU-only checks of the C ABI: the shared library loads, exports every symbol the header
declares, and its pure-host entry points (plan encoding, size queries, status strings)
behave as documented. No kernel is launched here.
"""
import ctypes as C
import os
import re

import numpy as np
import pytest

from jabas_amd import _lib as L

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "jabas_sync.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(jabas_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 15
    lib = L.lib()
    for n in names:
        assert hasattr(lib, n), f"{n} declared in jabas_sync.h but not exported"
    assert set(names) == set(L.SIGNATURES), "ctypes signature table and header disagree"


def test_struct_layouts_match_the_header():
    # sizes a C compiler gives the header's structs on x86-64 / amdgcn host ABI
    K = L.MAX_K
    assert K == 16 and L.STATS_STRIDE == 40 >= max(4 + K, 4 + 8 + 28)     # full rows of 16 VSWs, pair products of 8
    assert C.sizeof(L.JabasSpan) == K * 8 + 5 * 8 + (K - 1) * 8 + 8 + 6 * 4
    assert C.sizeof(L.JabasBound) == 16
    assert C.sizeof(L.JabasGroup) == 24
    assert C.sizeof(L.JabasStepArgs) == 4 + 4 + 4 * K + 4 + K + 4 * K + 4 * 4 + 4 + 5 * 8 + 16 * 24 + 8 + 8
    assert L.JabasStepArgs.scalars_dev.offset == C.sizeof(L.JabasStepArgs) - 8
    assert L.JabasStepArgs.groups.offset % 8 == 0 and L.JabasStepArgs.momentum.offset % 8 == 0


def test_version_and_status_strings():
    lib = L.lib()
    assert b"jabas_sync" in lib.jabas_sync_version()
    assert lib.jabas_status_string(0) == b"ok"
    seen = {lib.jabas_status_string(s) for s in range(-11, 0)}
    assert len(seen) == 11 and b"unknown status" not in seen
    assert lib.jabas_status_string(-99) == b"unknown status"


def _span(numel, base=0x7f0000000000, K=2, gs=4, skew=0, opt=False, stride=1 << 32):
    s = L.JabasSpan()
    for k in range(K):
        s.grads[k] = base + k * stride + skew * gs
    s.agg_out = base + 16 * stride + skew * 4
    if opt:
        s.param = base + 17 * stride + skew * 4
        s.state1 = base + 18 * stride + skew * 4
        s.state2 = base + 19 * stride + skew * 4
    s.numel = numel
    return s


def _encode(spans, bounds=(), K=2, dtype=L.F32, opt=L.OPT_NONE):
    lib = L.lib()
    arr = (L.JabasSpan * len(spans))(*spans)
    barr = (L.JabasBound * max(1, len(bounds)))()
    for i, (st, g) in enumerate(bounds):
        barr[i].start, barr[i].group = st, g
    nbytes = lib.jabas_plan_bytes(arr, len(spans), len(bounds), dtype)
    blob = np.zeros(nbytes // 8 + 1, dtype=np.uint64)
    rc = lib.jabas_plan_encode(arr, len(spans), barr if bounds else None, len(bounds), K, dtype, opt,
                               blob.ctypes.data, nbytes)
    return rc, blob, nbytes


def test_plan_encode_counts_chunks():
    """A tile is 1024 elements; a workgroup takes 2 tiles for K <= 4 and 4 tiles above."""
    lib = L.lib()
    sizes = [4096, 4097, 1, 0, 10 * 4096 + 5]
    rc, blob, _ = _encode([_span(n) for n in sizes])
    assert rc == L.OK
    assert lib.jabas_plan_chunks(blob.ctypes.data, 0) == 2 + 3 + 1 + 0 + 21
    assert lib.jabas_plan_chunks(blob.ctypes.data, 1) == 2 + 3 + 1 + 0 + 21      # K <= 4 without optimizer: one shape
    assert lib.jabas_plan_workspace_bytes(blob.ctypes.data) >= (27 + 5) * L.STATS_STRIDE * 8     # a row per chunk and per span, at least
    for K in (8, 16):                  # K > 4 without optimizer: 4 tiles of 1024 for both kinds of launch
        rc, blob, _ = _encode([_span(n, K=K) for n in sizes], K=K)
        assert rc == L.OK
        assert lib.jabas_plan_chunks(blob.ctypes.data, 1) == 1 + 2 + 1 + 0 + 11
        assert lib.jabas_plan_chunks(blob.ctypes.data, 0) == 1 + 2 + 1 + 0 + 11
    # a span that starts 3 elements into a 16-byte line needs one more tile when it is exactly full
    rc, blob, _ = _encode([_span(4096, skew=3)])
    assert rc == L.OK and lib.jabas_plan_chunks(blob.ctypes.data, 0) == 3


def test_plan_encode_starts_the_element_grid_at_a_256_byte_line_when_all_buffers_allow_it():
    """2048 elements per workgroup here (K = 2, no optimizer). With every buffer 61 elements into a
    256-byte line the grid starts at that line: 61 + 4036 elements still fit two workgroups, one
    more element does not. With one buffer elsewhere in its 256-byte line (but at the same place of
    its 16-byte line) the grid starts at the first element's 16-byte line, 1 element in."""
    lib = L.lib()
    for numel, want in ((4096 - 61, 2), (4096 - 60, 3)):
        rc, blob, _ = _encode([_span(numel, skew=61)])
        assert rc == L.OK and lib.jabas_plan_chunks(blob.ctypes.data, 0) == want
    for numel, want in ((4096 - 60, 2), (4095, 2), (4096, 3)):
        s = _span(numel, skew=61)
        s.agg_out -= 16 * 4                  # 45 elements in: congruent mod 4, not mod 64
        rc, blob, _ = _encode([s])
        assert rc == L.OK and lib.jabas_plan_chunks(blob.ctypes.data, 0) == want
    # the bound jabas_plan_bytes and jabas_sync_workspace_bytes are sized by holds in either case
    rc, blob, nbytes = _encode([_span(1, skew=63), _span(2048 - 63, skew=63), _span(2048 - 62, skew=63)])
    assert rc == L.OK and lib.jabas_plan_chunks(blob.ctypes.data, 0) == 1 + 1 + 2
    assert lib.jabas_sync_workspace_bytes(2048 - 62, L.F32) >= 3 * L.STATS_STRIDE * 8


def test_plan_encode_bf16_positions_are_counted_in_elements():
    # bf16 gradients 2 elements into an 8-byte line, fp32 buffers 2 elements into a 16-byte line: congruent
    rc, _, _ = _encode([_span(5000, gs=2, skew=2)], dtype=L.BF16)
    assert rc == L.OK
    s = _span(5000, gs=2, skew=2)
    s.agg_out += 4                      # now 3 elements in: not congruent with the gradients
    rc, _, _ = _encode([s], dtype=L.BF16)
    assert rc == L.ERR_ALIGN


def test_plan_encode_rejects_bad_spans():
    s = _span(4096)
    s.grads[1] += 4
    assert _encode([s])[0] == L.ERR_ALIGN                       # gradients not mutually congruent
    s = _span(4096)
    s.grads[1] = 0
    assert _encode([s])[0] == L.ERR_NULL
    assert _encode([_span(4096)], K=17)[0] == L.ERR_K
    assert _encode([_span(4096)], dtype=7)[0] == L.ERR_DTYPE
    assert _encode([_span(4096)], opt=9)[0] == L.ERR_OPT
    assert _encode([_span(4096)], opt=L.OPT_SGD)[0] == L.ERR_NULL    # optimizer without weights
    s = _span(4096, opt=True)
    s.state2 = 0
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_NULL
    assert _encode([s], opt=L.OPT_SGD)[0] == L.OK
    s = _span(4096)
    s.agg_out = s.grads[0] + 16                                 # overlaps VSW 0's buffer, not in place
    assert _encode([s])[0] == L.ERR_ALIAS
    s = _span(4096)
    s.agg_out = s.grads[0]                                      # exactly in place: allowed for fp32
    assert _encode([s])[0] == L.OK
    s = _span(4096, gs=2)
    s.agg_out = s.grads[0]
    assert _encode([s], dtype=L.BF16)[0] == L.ERR_ALIAS          # fp32 output over bf16 input
    s = _span(4096, opt=True)
    s.n_fanout = 16
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_SIZE


def test_plan_encode_checks_bounds():
    def with_bounds(bounds, count=None, begin=0):
        s = _span(10000, opt=True)
        s.bound_begin, s.bound_count = begin, len(bounds) if count is None else count
        return _encode([s], bounds=bounds, opt=L.OPT_SGD)[0]
    assert with_bounds([(0, 0), (100, 1), (9999, 0)]) == L.OK
    assert with_bounds([(1, 0)]) == L.ERR_GROUP                 # first bound must start at 0
    assert with_bounds([(0, 0), (100, 1), (100, 0)]) == L.ERR_GROUP   # not strictly increasing
    assert with_bounds([(0, 0), (10000, 1)]) == L.ERR_GROUP     # starts past the end
    assert with_bounds([(0, 16)]) == L.ERR_GROUP                # group index out of range
    assert with_bounds([(0, 0)], count=2) == L.ERR_GROUP        # table shorter than claimed


def test_plan_blob_too_small_and_garbage_header():
    lib = L.lib()
    spans = (L.JabasSpan * 1)(_span(4096))
    nbytes = lib.jabas_plan_bytes(spans, 1, 0, L.F32)
    blob = np.zeros(nbytes // 8 + 1, dtype=np.uint64)
    # jabas_plan_bytes is an upper bound over the launch shapes; the header and one span do not fit 128 bytes
    assert lib.jabas_plan_encode(spans, 1, None, 0, 2, L.F32, L.OPT_NONE, blob.ctypes.data, 128) == L.ERR_PLAN
    assert lib.jabas_plan_encode(spans, 1, None, 0, 2, L.F32, L.OPT_NONE, blob.ctypes.data, nbytes) == L.OK
    junk = np.zeros(64, dtype=np.uint64)
    assert lib.jabas_plan_chunks(junk.ctypes.data, 0) == L.ERR_PLAN
    assert lib.jabas_plan_workspace_bytes(junk.ctypes.data) == 0
    args = L.JabasStepArgs()
    args.K = 2
    assert lib.jabas_sync_fused(junk.ctypes.data, 0x1000, C.byref(args), None, None, 0, None) == L.ERR_PLAN
    assert lib.jabas_sync_fused(None, None, C.byref(args), None, None, 0, None) == L.ERR_NULL


def test_workspace_bytes_cover_any_line_position():
    lib = L.lib()
    row = L.STATS_STRIDE * 8
    assert lib.jabas_sync_workspace_bytes(0, L.F32) >= row
    assert lib.jabas_sync_workspace_bytes(4096, L.F32) >= 3 * row      # a shifted start adds a chunk
    assert lib.jabas_sync_workspace_bytes(1 << 30, L.BF16) >= ((1 << 30) // 2048) * row


def test_entry_points_validate_before_launching():
    """Argument errors are reported on a machine without a GPU because nothing is launched."""
    lib = L.lib()
    w = (C.c_float * 2)(0.5, 0.5)
    g = (C.c_void_p * 2)(0x7f0000000000, 0x7f0100000000)
    assert lib.jabas_aggregate(g, 0, L.F32, w, 0x7f0200000000, 100, None) == L.ERR_K
    assert lib.jabas_aggregate(g, 2, L.F32, w, None, 100, None) == L.ERR_NULL
    assert lib.jabas_aggregate(g, 2, 5, w, 0x7f0200000000, 100, None) == L.ERR_DTYPE
    g[1] = 0x7f0100000004
    assert lib.jabas_aggregate(g, 2, L.F32, w, 0x7f0200000000, 100, None) == L.ERR_ALIGN
    assert lib.jabas_sgd(None, 0x7f0000000000, None, 10, 0.1, 0.0, 0.0, 0.0, 0, 0, None) == L.ERR_NULL
    # momentum without a buffer
    assert lib.jabas_sgd(0x7f0000000000, 0x7f0100000000, None, 10, 0.1, 0.0, 0.9, 0.0, 0, 0, None) == L.ERR_NULL
    # nesterov needs momentum and zero dampening
    assert lib.jabas_sgd(0x7f0000000000, 0x7f0100000000, 0x7f0200000000, 10, 0.1, 0.0, 0.9, 0.1, 1, 0, None) == L.ERR_OPT
    # Adam's step count is 1-based
    assert lib.jabas_adam(0x7f0000000000, 0x7f0100000000, 0x7f0200000000, 0x7f0300000000, None, 10, 1e-3, 0.0, 0.9,
                          0.999, 1e-8, 0, 0, None) == L.ERR_OPT
    # amsgrad: the maximum is one more written buffer (it must not overlap the second moment), and its launches
    # take their scalars by value only
    assert lib.jabas_adam(0x7f0000000000, 0x7f0100000000, 0x7f0200000000, 0x7f0300000000, 0x7f0300000010, 10, 1e-3, 0.0,
                          0.9, 0.999, 1e-8, 1, 0, None) == L.ERR_ALIAS
    ams = L.JabasStepArgs()
    ams.K, ams.grad_dtype, ams.opt_kind, ams.n_groups = 1, L.F32, L.OPT_ADAMW_AMSGRAD, 1
    ams.weight[0], ams.beta1, ams.beta2, ams.eps = 1.0, 0.9, 0.999, 1e-8
    ams.groups[0].lr, ams.groups[0].step = 1e-3, 1
    sp = _span(1000, K=1, opt=True)
    assert lib.jabas_sync_bucket(C.byref(sp), None, C.byref(ams), None, None, 0, None) == L.ERR_NULL     # no state3
    block = np.zeros(L.STEP_SCALARS_BYTES, dtype=np.uint8)
    assert lib.jabas_step_scalars_encode(C.byref(ams), block.ctypes.data, block.nbytes) == L.ERR_OPT
    sp.state3 = 0x7f0000000000 + 21 * (1 << 32)
    ams.scalars_dev = 0x7f0000000000 + 22 * (1 << 32)
    assert lib.jabas_sync_bucket(C.byref(sp), None, C.byref(ams), None, None, 0, None) == L.ERR_OPT
    # statistics level 'gram' (pair products in the fused launch): up to STATS_GRAM_MAX_K workers; no level beyond it;
    # the static entry point's array holds rows of up to 4 + 16 sums and refuses the wider ones (six workers and more)
    many = L.JabasStepArgs()
    for dt, gs in ((L.F32, 4), (L.BF16, 2)):
        many.K, many.grad_dtype, many.stats = L.STATS_GRAM_MAX_K + 1, dt, L.STATS_GRAM
        spk = _span(1000, K=L.STATS_GRAM_MAX_K + 1, gs=gs)
        assert lib.jabas_sync_bucket(C.byref(spk), None, C.byref(many), 0x7f0400000000, 0x7f0500000000, 1 << 20, None) == L.ERR_K
        many.K = L.STATS_GRAM_MAX_K
        spk = _span(1000, K=L.STATS_GRAM_MAX_K, gs=gs)
        assert lib.jabas_sync_bucket(C.byref(spk), None, C.byref(many), 0x7f0400000000, 0x7f0500000000, 8, None) == L.ERR_WORKSPACE
        assert lib.jabas_sync_bucket_static(C.byref(spk), None, C.byref(many), 0x7f0400000000, None) == L.ERR_SIZE
        many.K = 6
        assert lib.jabas_sync_bucket_static(C.byref(_span(1000, K=6, gs=gs)), None, C.byref(many), 0x7f0400000000, None) == L.ERR_SIZE
    assert L.STAT_NORM_VSW0 + 8 + 28 == L.STATS_STRIDE == L.stat_pair(8, 6, 7) + 1
    many.K, many.stats = 2, L.STATS_GRAM + 1
    assert lib.jabas_sync_bucket(C.byref(spk), None, C.byref(many), 0x7f0400000000, 0x7f0500000000, 1 << 20, None) == L.ERR_OPT
    hid = (C.c_uint8 * 2)(0, 1)
    assert lib.jabas_stats(g, 2, L.F32, w, hid, w, 100, 0x7f0400000000, None, 0, None) == L.ERR_ALIGN
    g[1] = 0x7f0100000000
    assert lib.jabas_stats(g, 2, L.F32, w, hid, w, 100, 0x7f0400000000, None, 0, None) == L.ERR_WORKSPACE
    assert lib.jabas_gram(g, 2, L.F32, 100, 0x7f0400000000, None, 0, None) == L.ERR_WORKSPACE


def test_plain_c_client_sees_the_same_layout_and_drives_the_host_entry_points(tmp_path):
    """gcc -std=c99 compiles the header and a C client; the client links the library, reports the struct
    layout its compiler sees (compared field by field with the ctypes mirror) and encodes a plan."""
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    libdir = os.path.dirname(os.path.abspath(L.LIB_PATH))
    exe = str(tmp_path / "cabi_client")
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "cabi_client.c"), "-o", exe, "-L", libdir, "-ljabas_sync",
           "-Wl,-rpath," + libdir, "-Wl,--allow-shlib-undefined"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    out = subprocess.run([exe], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    seen = {}
    for line in out.stdout.splitlines():
        kind, name, *rest = line.split(" ", 2)
        seen[(kind, name)] = rest[0] if rest else ""
    structs = {"JabasSpan": L.JabasSpan, "JabasBound": L.JabasBound, "JabasGroup": L.JabasGroup,
               "JabasStepArgs": L.JabasStepArgs}
    checked = 0
    for (kind, name), val in seen.items():
        if kind == "sizeof":
            assert C.sizeof(structs[name]) == int(val), name
            checked += 1
        elif kind == "offsetof":
            s, f = name.split(".")
            assert getattr(structs[s], f).offset == int(val), name
            checked += 1
    assert checked == 40
    # every field of the ctypes mirror was reported by the C side (reserved words aside)
    for sname, st in structs.items():
        for f, _ in st._fields_:
            if not f.startswith("reserved") and not f.startswith("_"):
                assert ("offsetof", f"{sname}.{f}") in seen, f"{sname}.{f}"
    assert seen[("version", "jabas_sync")].startswith("0.")
    assert seen[("status0", "ok")] == ""
    assert seen[("encode", "0")] == ""
    assert seen[("chunks", "14")] == ""                      # SGD, K = 2, fp32, plain: 1024 elements per chunk -> 5 + 9
    assert seen[("chunks_stats", "8")] == ""                 # with statistics: 2048 per chunk -> 3 + 5
    assert int(next(n for (k, n) in seen if k == "workspace")) >= (8 + 2) * L.STATS_STRIDE * 8
    assert ("encode_misaligned", str(L.ERR_ALIGN)) in seen
    # the ctypes mirror places the pair products of a 'gram' row where the header's macro does: behind the K norms,
    # in the order (0,1), (0,2), ..., (K-2,K-1), and within the row's JABAS_STATS_STRIDE slots
    for K, key in ((4, "pairs4"), (3, "pairs3")):
        want = [L.stat_pair(K, a, b) for a in range(K) for b in range(a + 1, K)]
        assert ("pairs%d" % K, ",".join(map(str, want))) in seen
        assert want == list(range(4 + K, 4 + K + K * (K - 1) // 2)) and want[-1] < L.STATS_STRIDE


def test_plan_encode_checks_interleaved_moments():
    """A span whose Adam moments sit interleaved in one arena (state_block_log2): the layout rules, and the
    moments from the first element's exp_avg to the last element's last moment as ONE written range."""
    T, n = 1 << 10, 5000
    arena = 0x7f0000000000 + 40 * (1 << 32)

    def span(pos=0, first_block=0, ways=2):
        s = _span(n, opt=True)
        s.state1 = arena + 4 * (first_block * ways * T + pos)
        s.state2 = s.state1 + 4 * T
        s.state3 = s.state1 + 8 * T if ways == 3 else None
        s.state_block_log2, s.state_block_pos = 10, pos
        return s
    assert _encode([span()], opt=L.OPT_ADAM)[0] == L.OK
    assert _encode([span()], opt=L.OPT_ADAMW)[0] == L.OK
    assert _encode([span(ways=3)], opt=L.OPT_ADAM_AMSGRAD)[0] == L.OK
    assert _encode([span()], opt=L.OPT_ADAM_AMSGRAD)[0] == L.ERR_NULL          # the maximum has no place in a two-way arena
    assert _encode([span()], opt=L.OPT_SGD)[0] == L.ERR_OPT
    s = span()
    s.state_block_log2 = 7
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_SIZE
    s = span()
    s.state_block_log2 = 25
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_SIZE
    s = span()
    s.state_block_pos = T
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_SIZE
    s = span()
    s.state2 += 16
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIGN
    s = span(ways=3)
    s.state3 -= 4 * T
    assert _encode([s], opt=L.OPT_ADAM_AMSGRAD)[0] == L.ERR_ALIGN
    s = span()
    s.state_block_pos = 2                                         # the block group would start 8 bytes off a 16-byte line
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIGN
    # a span in the middle of a block, at the other buffers' element of a 16-byte line
    s = _span(n, opt=True, skew=3)
    s.state1 = arena + 4 * (2 * T + 64 * 3 + 3)
    s.state2, s.state_block_log2, s.state_block_pos = s.state1 + 4 * T, 10, 64 * 3 + 3
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.OK
    s.state_block_pos -= 1                                        # another element of the line than the weights'
    s.state1 -= 4
    s.state2 -= 4
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIGN
    # 5000 elements from position 0: blocks 0..4 of exp_avg and of exp_avg_sq, the last ends 4 * (9 * T + 904) bytes in
    end = arena + 4 * (9 * T + n - 4 * T)
    s = span()
    s.param = end                                                 # right behind the last second moment: fine
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.OK
    s.param = end - 16
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIAS
    s = span()
    s.agg_out = arena + 4 * T + 256                               # inside the first block of second moments
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIAS
    s = span()
    s.grads[1] = arena + 4 * (3 * T)                              # a gradient buffer inside a block the span does not own
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIAS         # ... but which lies inside the one written range


def test_plan_encode_rejects_overlapping_written_buffers():
    def span():
        return _span(4096, opt=True)
    s = span()
    s.state1 = s.param + 4096 * 4 - 16                          # last four weights = first four momentum entries
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_ALIAS
    s = span()
    s.state1 = s.param + 4096 * 4                               # back to back: fine
    assert _encode([s], opt=L.OPT_SGD)[0] == L.OK
    s = span()
    s.state2 = s.state1
    assert _encode([s], opt=L.OPT_ADAM)[0] == L.ERR_ALIAS
    assert _encode([s], opt=L.OPT_SGD)[0] == L.OK               # SGD never touches state2
    s = span()
    s.param = s.grads[1]                                        # weights over a worker's gradients
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_ALIAS
    s = span()
    s.param = s.agg_out
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_ALIAS
    s = span()
    s.n_fanout = 2
    s.fanout[0] = s.param + (1 << 30)
    s.fanout[1] = s.fanout[0] + 16
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_ALIAS
    s.fanout[1] = s.fanout[0] + 4096 * 4
    assert _encode([s], opt=L.OPT_SGD)[0] == L.OK
    s.fanout[1] = s.param
    assert _encode([s], opt=L.OPT_SGD)[0] == L.ERR_ALIAS
    s = span()
    s.param = s.grads[0]                                        # ignored without an optimizer
    assert _encode([s], opt=L.OPT_NONE)[0] == L.OK


def test_launch_shape_follows_what_the_plan_is_encoded_for():
    """Launches with full statistics rows run 256-thread workgroups of 2 tiles (K <= 4) or 4 tiles, with
    similarity sums only 2 tiles for every K; plain launches with an optimizer 256 threads x 2 tiles for K > 4,
    128 threads x 2 tiles for SGD with fp32 gradients and K <= 4, 256 x 4 for the Adam kinds and K <= 4, else 256 x 2;
    aggregate-only launches 256 x 2 (K <= 4) or 256 x 4. A plan holds a chunk table per shape and serves launches of its own optimizer class only."""
    lib = L.lib()
    n = 10 * 4096
    def chunks(K, dtype, opt, gs=4):
        rc, blob, _ = _encode([_span(n, K=K, gs=gs, opt=True)], K=K, dtype=dtype, opt=opt)
        assert rc == L.OK
        return (lib.jabas_plan_chunks(blob.ctypes.data, 0), lib.jabas_plan_chunks(blob.ctypes.data, 1)), blob
    assert chunks(2, L.F32, L.OPT_SGD)[0] == (n // 1024, n // 2048)
    assert chunks(4, L.F32, L.OPT_SGD)[0] == (n // 1024, n // 2048)
    assert chunks(5, L.F32, L.OPT_SGD)[0] == (n // 2048, n // 4096)
    assert chunks(2, L.BF16, L.OPT_SGD, gs=2)[0] == (n // 2048, n // 2048)
    assert chunks(2, L.F32, L.OPT_ADAM)[0] == (n // 4096, n // 2048)
    assert chunks(8, L.BF16, L.OPT_ADAMW, gs=2)[0] == (n // 2048, n // 4096)
    assert chunks(2, L.F32, L.OPT_NONE)[0] == (n // 2048, n // 2048)
    assert chunks(8, L.F32, L.OPT_NONE)[0] == (n // 4096, n // 4096)
    _, blob8 = chunks(8, L.BF16, L.OPT_ADAMW, gs=2)
    assert lib.jabas_plan_chunks(blob8.ctypes.data, L.STATS_SIMILARITY) == n // 2048
    _, blob2 = chunks(2, L.F32, L.OPT_SGD)
    assert lib.jabas_plan_chunks(blob2.ctypes.data, L.STATS_SIMILARITY) == n // 2048
    # the level with pair products launches in the shape of the full rows and uses their chunk table
    assert lib.jabas_plan_chunks(blob2.ctypes.data, L.STATS_GRAM) == lib.jabas_plan_chunks(blob2.ctypes.data, L.STATS_FULL)
    assert lib.jabas_plan_chunks(blob2.ctypes.data, L.STATS_GRAM + 1) == L.ERR_OPT
    _, blob = chunks(2, L.F32, L.OPT_SGD)
    assert lib.jabas_plan_workspace_bytes(blob.ctypes.data) >= (n // 2048 + 1) * L.STATS_STRIDE * 8
    args = L.JabasStepArgs()
    args.K, args.grad_dtype, args.opt_kind = 2, L.F32, L.OPT_NONE
    assert lib.jabas_sync_fused(blob.ctypes.data, 0x1000, C.byref(args), None, None, 0, None) == L.ERR_PLAN
    args.opt_kind, args.n_groups = L.OPT_ADAM, 1
    args.groups[0].step = 1
    assert lib.jabas_sync_fused(blob.ctypes.data, 0x1000, C.byref(args), None, None, 0, None) == L.ERR_PLAN


def test_product_paths_fail_when_the_library_is_missing(tmp_path):
    """No CPU fallback: with no shared library the loader raises, and product entries given host
    tensors refuse them or raise the loader's error; none computes anything (checked in a child
    process so that this process keeps its loaded library)."""
    import subprocess
    import sys
    code = """
import torch
from jabas_amd import _lib, sync
from jabas_amd.local_sync import LocalBucketSync
g = [torch.ones(8), torch.ones(8)]
for name, call in (("lib", lambda: _lib.lib()),
                   ("aggregate", lambda: sync.aggregate(g, (1, 1))),
                   ("gradient_stats", lambda: sync.gradient_stats(g, (1, 1))),
                   ("plan", lambda: sync.SyncPlan([sync.SpanSpec(g, agg_out=torch.zeros(8))], _lib.OPT_NONE))):
    try:
        call()
    except (RuntimeError, ValueError) as exc:
        assert "no CPU fallback" in str(exc) or (name != "lib" and "must live on the GPU" in str(exc)), (name, exc)
    else:
        raise SystemExit(name + " did not raise")
print("all raised")
"""
    env = dict(os.environ, JABAS_SYNC_LIB=str(tmp_path / "absent.so"))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, "-c", code], cwd=root, env=env, capture_output=True, text=True, timeout=300)
    assert res.returncode == 0 and "all raised" in res.stdout, res.stdout + res.stderr


def test_statistics_over_too_many_spans_are_refused_before_any_launch():
    """The finalize launch indexes spans by a grid dimension of 16 bits; a plan beyond that must be
    turned down with a status, not fail after the weights have moved."""
    lib = L.lib()
    n_span = 65536
    arr = (L.JabasSpan * n_span)()
    base = 0x7f0000000000
    for i in range(n_span):
        arr[i].grads[0] = base + 4096 * i
        arr[i].grads[1] = base + (1 << 36) + 4096 * i
        arr[i].agg_out = base + (2 << 36) + 4096 * i
        arr[i].numel = 8
    nbytes = lib.jabas_plan_bytes(arr, n_span, 0, L.F32)
    blob = np.zeros(nbytes // 8 + 1, dtype=np.uint64)
    assert lib.jabas_plan_encode(arr, n_span, None, 0, 2, L.F32, L.OPT_NONE, blob.ctypes.data, nbytes) == L.OK
    args = L.JabasStepArgs()
    args.K, args.grad_dtype, args.opt_kind, args.stats = 2, L.F32, L.OPT_NONE, 1
    args.weight[0] = args.weight[1] = 0.5
    args.half_id[1] = 1
    args.half_weight[0] = args.half_weight[1] = 1.0
    fake_dev = 0x7e0000000000
    ws_bytes = lib.jabas_plan_workspace_bytes(blob.ctypes.data)
    rc = lib.jabas_sync_fused(blob.ctypes.data, fake_dev, C.byref(args), fake_dev + (1 << 30), fake_dev + (2 << 30),
                              ws_bytes, None)
    assert rc == L.ERR_SIZE


def _shape_model(K, dtype, opt_class, stats):
    """(threads per workgroup, tiles per workgroup) as documented for the launch shapes."""
    if stats or opt_class == 0 or K > 4:
        block = 256
    else:
        block = 128 if (opt_class == 1 and dtype == L.F32) else 256
    if K > 4:
        tiles = 2 if stats == 2 else (4 if (stats or opt_class == 0) else 2)
    else:
        tiles = 4 if (not stats and opt_class >= 2) else 2
    return block, tiles


@pytest.mark.parametrize("seed", range(40))
def test_plan_encode_against_a_python_statement_of_the_chunking_rule(seed):
    """Random spans at random addresses: the encoder's verdict (OK / JABAS_ERR_ALIGN) and its chunk
    counts for both launch shapes must equal an independent statement of the rule: buffers must agree
    within 4 elements; the element grid starts at the 256-byte line when they agree within 64 elements,
    else at the 16-byte line; a span takes ceil(ceil((skew + numel) / tile) / tiles_per_workgroup) chunks."""
    rng = np.random.RandomState(seed)
    lib = L.lib()
    K = int(rng.randint(1, 17))
    dtype = L.BF16 if rng.rand() < 0.4 else L.F32
    opt = [L.OPT_NONE, L.OPT_SGD, L.OPT_ADAM, L.OPT_ADAMW][int(rng.randint(0, 4))]
    opt_class = {L.OPT_NONE: 0, L.OPT_SGD: 1, L.OPT_ADAM: 2, L.OPT_ADAMW: 2}[opt]
    gs = 2 if dtype == L.BF16 else 4
    n_span = int(rng.randint(1, 12))
    spans, want_chunks, want_rc = [], [0, 0, 0], L.OK
    stride = 1 << 36
    for i in range(n_span):
        numel = int(rng.choice([0, 1, 3, 500, 1023, 1024, 1025, 4096, 4097, 70000, 1 << 20])) + int(rng.randint(0, 3))
        mode = rng.rand()
        base_off = int(rng.randint(0, 64))
        n_buf = K + 4
        if mode < 0.6:
            offs = [base_off] * n_buf                                   # one place within the 256-byte line
        elif mode < 0.9:
            offs = [base_off % 4 + 4 * int(rng.randint(0, 16)) for _ in range(n_buf)]   # agree within 16 bytes only
        else:
            offs = [int(rng.randint(0, 64)) for _ in range(n_buf)]      # arbitrary
        s = L.JabasSpan()
        region = (2 * i + 1) * (1 << 28)                                # spans far apart: no overlap between buffers
        for k in range(K):
            s.grads[k] = 0x700000000000 + k * stride + region + offs[k] * gs
        s.agg_out = 0x700000000000 + 16 * stride + region + offs[K] * 4
        used = offs[:K + 1]
        if opt_class:
            s.param = 0x700000000000 + 17 * stride + region + offs[K + 1] * 4
            s.state1 = 0x700000000000 + 18 * stride + region + offs[K + 2] * 4
            used = offs[:K + 3]
            if opt_class == 2:
                s.state2 = 0x700000000000 + 19 * stride + region + offs[K + 3] * 4
                used = offs[:K + 4]
        s.numel = numel
        spans.append(s)
        if numel == 0:
            continue
        if len({o % 4 for o in used}) != 1:
            want_rc = L.ERR_ALIGN
            continue
        skew = used[0] if len(set(used)) == 1 else used[0] % 4
        for v, stats in enumerate((0, 1, 2)):                           # statistics level of the launch
            block, tiles = _shape_model(K, dtype, opt_class, stats)
            te = block * 4
            want_chunks[v] += -(-(-(-(skew + numel) // te)) // tiles)
    arr = (L.JabasSpan * n_span)(*spans)
    nbytes = lib.jabas_plan_bytes(arr, n_span, 0, dtype)
    blob = np.zeros(nbytes // 8 + 1, dtype=np.uint64)
    rc = lib.jabas_plan_encode(arr, n_span, None, 0, K, dtype, opt, blob.ctypes.data, nbytes)
    if want_rc != L.OK:
        assert rc == L.ERR_ALIGN
        return
    assert rc == L.OK, rc
    assert lib.jabas_plan_chunks(blob.ctypes.data, 0) == want_chunks[0]
    assert lib.jabas_plan_chunks(blob.ctypes.data, 1) == want_chunks[1]
    assert lib.jabas_plan_chunks(blob.ctypes.data, 2) == want_chunks[2]
    assert lib.jabas_plan_chunks(blob.ctypes.data, 3) == want_chunks[1]        # pair products: the shape of the full rows
    assert lib.jabas_plan_chunks(blob.ctypes.data, 4) == L.ERR_OPT


def test_rendezvous_calls_validate_their_arguments():
    """The meeting point's argument checks (no GPU: creating the object itself needs a device and is covered by
    the GPU tests)."""
    lib = L.lib()
    h = C.c_void_p()
    assert lib.jabas_rdv_create(0, C.byref(h)) == L.ERR_K and not h.value
    assert lib.jabas_rdv_create(L.MAX_K + 1, C.byref(h)) == L.ERR_K
    assert lib.jabas_rdv_create(2, None) == L.ERR_NULL
    args, span = L.JabasStepArgs(), L.JabasSpan()
    assert lib.jabas_rdv_publish(None, 0, 0, 0, None, None, C.byref(args), L.STATS_SIMILARITY) == L.ERR_NULL
    assert lib.jabas_rdv_set_bucket(None, 0, C.byref(span), None, None, None, 0, 0) == L.ERR_NULL
    assert lib.jabas_rdv_drop_bucket(None, 0) == L.ERR_NULL
    assert lib.jabas_rdv_reset(None) == L.ERR_NULL
    lib.jabas_rdv_destroy(None)
    assert b"rendezvous" in lib.jabas_status_string(L.ERR_STATE)


def test_step_scalar_block_holds_the_constants_a_plain_call_derives():
    """jabas_step_scalars_encode is host code: its block is compared, slot by slot, with the constants derived
    here in Python doubles and rounded once to fp32 (what a Python float becomes as an fp32 kernel scalar)."""
    import torch
    from jabas_amd import sync
    lib = L.lib()
    f32 = lambda x: np.float32(x)
    opt = dict(kind="adamw", betas=(0.9, 0.999), eps=1e-8,
               groups=[dict(lr=5e-4, weight_decay=0.05, step=7), dict(lr=1e-3, weight_decay=0.0, step=3)])
    batches = (48, 32, 32, 16, 8)
    m = 2.5 ** 0.5
    args = sync.make_step_args(batches, torch.bfloat16, stats="similarity", opt=opt, lr_scale=m,
                               half_id=[0, 1, 1, 0, 1])
    block = np.zeros(L.STEP_SCALARS_BYTES, dtype=np.uint8)
    assert lib.jabas_step_scalars_encode(C.byref(args), block.ctypes.data, block.nbytes) == L.OK
    fl, u32 = block.view(np.float32), block.view(np.uint32)
    w, hid, hw = sync.batch_weights(batches, [0, 1, 1, 0, 1])
    assert np.array_equal(fl[0:5], w) and not fl[5:16].any()
    assert np.array_equal(fl[16:21], hw) and not fl[21:32].any()
    o = 32                                                       # OptDev: 7 floats, 4 flags
    assert fl[o + 2] == f32(0.9) and fl[o + 3] == f32(1.0 - 0.9)
    assert fl[o + 4] == f32(0.999) and fl[o + 5] == f32(1.0 - 0.999) and fl[o + 6] == f32(1e-8)
    assert list(u32[o + 7:o + 11]) == [0, 0, 0, 1]               # has_momentum, first_step, nesterov, adamw
    assert u32[o + 11] == 0b10110                                # half B: workers 1, 2, 4
    for i, g in enumerate(opt["groups"]):
        base = 44 + 8 * i
        lr = g["lr"] * m
        assert fl[base + 0] == f32(g["weight_decay"])
        assert fl[base + 1] == f32(-lr)
        assert fl[base + 2] == f32(1.0 - lr * g["weight_decay"])
        assert fl[base + 3] == f32(-(lr / (1.0 - 0.9 ** g["step"])))
        assert fl[base + 4] == f32((1.0 - 0.999 ** g["step"]) ** 0.5)
    assert not fl[44 + 16:].any()
    # SGD: momentum, dampening, the first-step flag
    sgd = dict(kind="sgd", momentum=0.9, dampening=0.1, nesterov=False, groups=[dict(lr=0.1, weight_decay=1e-4)])
    args = sync.make_step_args((2, 2), torch.float32, opt=sgd, first_step=True)
    assert lib.jabas_step_scalars_encode(C.byref(args), block.ctypes.data, block.nbytes) == L.OK
    assert fl[o] == f32(0.9) and fl[o + 1] == f32(1.0 - 0.1) and list(u32[o + 7:o + 11]) == [1, 1, 0, 0]
    assert fl[44 + 1] == f32(-0.1) and fl[44 + 3] == 0.0 and fl[44 + 4] == 1.0
    # argument checks
    assert lib.jabas_step_scalars_encode(None, block.ctypes.data, block.nbytes) == L.ERR_NULL
    assert lib.jabas_step_scalars_encode(C.byref(args), None, block.nbytes) == L.ERR_NULL
    assert lib.jabas_step_scalars_encode(C.byref(args), block.ctypes.data, L.STEP_SCALARS_BYTES - 1) == L.ERR_SIZE
    none = sync.make_step_args((2, 2), torch.float32)
    assert lib.jabas_step_scalars_encode(C.byref(none), block.ctypes.data, block.nbytes) == L.ERR_OPT
    adam0 = sync.make_step_args((2, 2), torch.float32, opt=dict(opt, groups=[dict(lr=1e-3, step=0)]))
    assert lib.jabas_step_scalars_encode(C.byref(adam0), block.ctypes.data, block.nbytes) == L.ERR_OPT
    assert lib.jabas_step_scalars_upload(None, 0x7f0000001000, None) == L.ERR_NULL
    assert lib.jabas_step_scalars_upload(C.byref(args), None, None) == L.ERR_NULL
    assert lib.jabas_step_scalars_upload(C.byref(args), 0x7f0000001004, None) == L.ERR_ALIGN
    assert lib.jabas_step_scalars_upload(C.byref(none), 0x7f0000001000, None) == L.ERR_OPT
    # a launch without optimizer has nothing that moves between steps: a block is refused, as is a misaligned one
    span = _span(5000)
    none.scalars_dev = 0x7f0000001000
    assert lib.jabas_sync_bucket(C.byref(span), None, C.byref(none), None, None, 0, None) == L.ERR_OPT
    span = _span(5000, opt=True)
    args.scalars_dev = 0x7f0000001008
    assert lib.jabas_sync_bucket(C.byref(span), None, C.byref(args), None, None, 0, None) == L.ERR_ALIGN
