"""Host logic of the interleaved moment arena (``sync.MomentArena``) on CPU tensors: where an element's
moments sit, flat reads and writes across block boundaries, and what a span names as its place in the arena."""
import ctypes as C

import pytest
import torch

from jabas_amd import _lib as L
from jabas_amd import sync


@pytest.mark.parametrize("ways", [2, 3])
def test_layout_reads_and_writes(ways):
    T, n = 256, 1000
    a = sync.MomentArena(n, ways, "cpu", 8)
    assert a.T == T and a.blocks == 4 and a.buf.numel() == 4 * ways * T and a.buf.data_ptr() % 256 == 0
    x = [torch.arange(n, dtype=torch.float32) * (j + 1) + 0.5 for j in range(ways)]
    for j in range(ways):
        a.write(j, x[j])
    for j in range(ways):
        assert torch.equal(a.read(j), x[j])
        for i in (0, 1, 255, 256, 257, 511, 512, 999):          # element i of moment j: i + (ways - 1)(i - i mod T) + jT
            assert a.buf[i + (ways - 1) * (i - i % T) + j * T].item() == x[j][i].item()
        assert torch.equal(a.read(j, 250, 10), x[j][250:260])             # across a block boundary
        assert torch.equal(a.read(j, 300, 600), x[j][300:900])            # across several
        assert torch.equal(a.read(j, 10, 5), x[j][10:15])                 # inside one block
        assert a.read(j, 5, 0).numel() == 0
        assert torch.equal(a.way(j).reshape(-1)[:n], x[j])
    a.write(ways - 1, torch.full((5,), -1.0), 254)                        # two elements in block 0, three in block 1
    assert a.read(ways - 1, 253, 7).tolist() == [x[ways - 1][253].item(), -1, -1, -1, -1, -1, x[ways - 1][259].item()]
    assert torch.equal(a.read(0), x[0])                                   # the other moments untouched
    got = a.read(0, 700, 50)
    got.zero_()                                                           # reads are copies, also inside one block
    assert torch.equal(a.read(0, 700, 50), x[0][700:750])
    with pytest.raises(ValueError):
        a.write(0, torch.zeros(10), 4 * T - 5)
    with pytest.raises(ValueError):
        sync.MomentArena(10, 4, "cpu")
    with pytest.raises(ValueError):
        sync.MomentArena(10, 2, "cpu", 7)


def test_a_spans_place_in_the_arena():
    a = sync.MomentArena(5000, 2, "cpu", 10)
    base = a.buf.data_ptr()
    assert a.place(0) == (base, 0)
    assert a.place(1023) == (base + 4 * 1023, 1023)
    assert a.place(1024) == (base + 4 * 2048, 0)                          # block 1 of exp_avg starts behind block 0 of exp_avg_sq
    assert a.place(2500) == (base + 4 * (2 * 2048 + 452), 452)
    b = sync.MomentArena(5000, 3, "cpu", 10)
    assert b.place(2500) == (b.buf.data_ptr() + 4 * (2 * 3072 + 452), 452)


def test_span_spec_names_the_arena_or_the_tensors_not_both():
    a = sync.MomentArena(100, 2, "cpu", 8)
    g = [torch.zeros(10)]
    with pytest.raises(ValueError, match="one or the other"):
        sync.SpanSpec(g, param=torch.zeros(10), state1=torch.zeros(10), moments=(a, 0))
    assert L.JabasSpan.state_block_log2.offset + 4 == L.JabasSpan.state_block_pos.offset
    assert C.sizeof(L.JabasSpan) % 8 == 0
    assert sync.MOMENT_BLOCK_LOG2 == 13
