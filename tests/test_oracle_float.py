"""Pins the row-movement, FFN, combine and fp8 oracles against definitions that
do not share their code: row loops, torch library routines, fp64 arithmetic."""
import numpy as np
import pytest
import torch

from oracle import ffn, fp8, routing, rows


def test_permute_matches_reference_test_loop():
    # the case of tests/ops/test_memory.py:8-31: 64 x 4096 bf16, ids in [2, 8)
    g = torch.Generator().manual_seed(0)
    t = torch.randn(64, 4096, generator=g).to(torch.bfloat16)
    ids = torch.randint(2, 8, (64,), generator=g)
    m, _ = routing.get_mappings_from_exp_ids(ids, 8)
    std = torch.empty_like(t)
    for i in range(64):
        std[m[i], :] = t[i, :]
    assert torch.equal(rows.permute_tokens(t, m), std)


@pytest.mark.parametrize("k", [1, 2, 6])
def test_permute_topk_is_repeat_then_index_select(k):
    g = torch.Generator().manual_seed(k)
    T, d, E = 37, 64, 5
    t = torch.randn(T, d, generator=g).to(torch.float16)
    ids = torch.randint(0, E, (T * k,), generator=g)
    m, _ = routing.get_mappings_from_exp_ids(ids, E)
    inv = torch.empty(T * k, dtype=torch.int64)
    inv[torch.tensor(m)] = torch.arange(T * k)
    expect = torch.index_select(t.repeat_interleave(k, 0), 0, inv)
    assert torch.equal(rows.permute_tokens(t, m), expect)
    assert torch.equal(rows.gather_rows(t, inv // k), expect)


def test_gather_row_slabs():
    g = torch.Generator().manual_seed(3)
    slabs = [torch.randn(n, 16, generator=g).to(torch.bfloat16) for n in (3, 0, 5)]
    ids = [[1, 0, 1], [], [0, 2, 2, 1, 0]]
    m, cnt = routing.merge_by_exp_ids(ids, 3)
    out = rows.gather_row_slabs(slabs, m)
    stream = torch.cat(slabs)
    flat = [v for b in ids for v in b]
    for s, dst in enumerate(m):
        assert torch.equal(out[dst], stream[s])
    assert [flat[m.index(r)] for r in range(8)] == sorted(flat)


def test_gmm_single_expert_is_matmul():
    g = torch.Generator().manual_seed(1)
    a = torch.randn(33, 48, generator=g).to(torch.bfloat16)
    b = torch.randn(1, 48, 40, generator=g).to(torch.bfloat16)
    out = ffn.gmm(a, b, torch.tensor([33]))
    assert torch.equal(out, (a.float() @ b[0].float()).to(torch.bfloat16))
    out_t = ffn.gmm(a, b.transpose(1, 2).contiguous(), [33], trans_b=True)
    assert torch.equal(out_t, out)


def test_gmm_ragged_against_fp64_blocks():
    g = torch.Generator().manual_seed(2)
    sizes = [0, 5, 0, 1, 9, 0]
    R = sum(sizes) + 3                       # three rows past the end stay untouched
    a = torch.randn(R, 24, generator=g).to(torch.bfloat16)
    b = torch.randn(len(sizes), 24, 16, generator=g).to(torch.bfloat16)
    c = torch.full((R, 16), 7.0, dtype=torch.bfloat16)
    out = ffn.gmm(a, b, sizes, c=c)
    assert out is c
    o = 0
    for e, n in enumerate(sizes):
        blk = (a[o:o + n].double() @ b[e].double())
        assert torch.allclose(out[o:o + n].double(), blk, rtol=2 ** -8, atol=1e-6)
        o += n
    assert (out[o:] == 7.0).all()
    assert ffn.gmm(a, b, [0] * 6, c=torch.zeros(R, 16, dtype=torch.bfloat16)).abs().sum() == 0


def test_ffn_against_serial_fp64():
    g = torch.Generator().manual_seed(4)
    E, d, I = 3, 32, 24
    sizes = [4, 0, 7]
    x = torch.randn(sum(sizes), d, generator=g).to(torch.bfloat16)
    w13 = (torch.randn(E, d, 2 * I, generator=g) * 0.2).to(torch.bfloat16)
    w2 = (torch.randn(E, I, d, generator=g) * 0.2).to(torch.bfloat16)
    out = ffn.moe_experts_forward(x, w13, w2, sizes)
    o = 0
    for e, n in enumerate(sizes):
        xe = x[o:o + n].double()
        w1, w3 = w13[e, :, :I].double(), w13[e, :, I:].double()
        gate = xe @ w1
        ref = (gate / (1 + torch.exp(-gate)) * (xe @ w3)) @ w2[e].double()
        assert torch.allclose(out[o:o + n].double(), ref, rtol=2 ** -7, atol=1e-3)
        o += n
    chain = ffn.moe_experts_forward_reference_rounding(x, w13, w2, sizes)
    assert ffn.max_rel_err(chain, out) < 1e-2


def test_combine_closed_form_and_chain():
    g = torch.Generator().manual_seed(5)
    T, k, d, E = 9, 2, 16, 4
    ids = torch.randint(0, E, (T, k), generator=g)
    m, _ = routing.get_mappings_from_exp_ids(ids, E)
    y = torch.randn(T * k, d, generator=g).to(torch.bfloat16)
    w = torch.softmax(torch.randn(T, k, generator=g), dim=1)
    out = ffn.combine(y, m, w)
    for i in range(T):
        ref = sum(w[i, j].double() * y[m[i * k + j]].double() for j in range(k))
        assert torch.allclose(out[i].double(), ref, rtol=2 ** -8, atol=1e-6)
    # the reference's statements: scale (engine.py:731-732), permute back to k-major, add halves (:627)
    scaled = y * w.to(torch.bfloat16).view(-1)[torch.argsort(torch.tensor(m))].view(-1, 1)
    back = torch.empty_like(scaled)
    inv = torch.argsort(torch.tensor(m))          # sorted row -> flat t
    for r in range(T * k):
        t = int(inv[r])
        back[(t % k) * T + t // k] = scaled[r]    # k-major layout j*T + i
    expect = back[:T] + back[T:]
    assert torch.equal(ffn.combine_reference_chain(y, m, w), expect)


def test_fp8_quantisation_rules():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(17, 64, generator=g).to(torch.bfloat16)
    x[3] = 0
    q, s = fp8.quantize_rows(x)
    assert q.dtype == torch.float8_e4m3fn and s.dtype == torch.float32
    assert s[3] == 1 and (q[3].float() == 0).all()
    amax = x.float().abs().amax(dim=1)
    assert torch.equal(s[amax > 0], (amax / 448.0)[amax > 0])
    assert q.float().abs().max() <= 448
    back = fp8.dequantize_rows(q, s, torch.float32)
    # e4m3 keeps 3 mantissa bits: relative error <= 2^-4 for normal values
    big = x.float().abs() > (s[:, None] * 2 ** -6)
    assert ((back - x.float()).abs()[big] <= x.float().abs()[big] * 2 ** -4 + 1e-12).all()
    w = (torch.randn(2, 32, 24, generator=g) * 0.02).to(torch.bfloat16)
    qw, sw = fp8.quantize_weight_channels(w)
    assert qw.shape == (2, 24, 32) and sw.shape == (2, 24)
    assert torch.equal(sw, w.float().abs().amax(dim=1) / 448.0)
    dq = fp8.dequantize_weight(qw, sw, torch.float32)
    assert dq.shape == w.shape and ffn.max_rel_err(dq, w.float()) < 2 ** -4
