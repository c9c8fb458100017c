"""Pins oracle/fp8.py:moe_experts_forward_fp8 (the checker of the fp8 bar) and
oracle/cpu_path.py (the cpu_baseline leg) on the CPU, by cases whose answers do
not come from the oracle's own formula:

* inputs that already lie on the e4m3 grid with a power-of-two scale, built so that
  every quantisation point of the fp8 FFN is the identity: the result must be the
  bits of the unquantised fp32 FFN oracle on the same values;
* a hand-computed case in which the quantisation of the intermediate row changes
  the result (so leaving that step out, or scaling by the wrong axis, fails);
* zero rows, zero-size experts;
* cpu_path against the stage-by-stage oracles.
"""
import torch

from oracle import cpu_path, ffn, fp8, routing, rows

# e4m3fn values with exponent 0..8 (1 .. 448): 4 significant bits
_GRID = sorted({(8 + m) * 2.0 ** (e - 3) for e in range(0, 9) for m in range(8) if (8 + m) * 2.0 ** (e - 3) <= 448})


def _on_grid_case(E=3, sel=5, I=6, d_out=4, sizes=(4, 0, 3), seed=0):
    """Rows, weights and sizes for which every quantisation in the fp8 FFN is exact.

    x[r] = 2^p at one selector column c(r), 448 * 2^a at column `sel` (sets the row scale to 2^a), 0 at column
    sel + 1.  w13[e][sel] = 0, w13[e][sel + 1] = 448 * 2^b in every column (sets every channel scale to 2^b, never
    contracted because x is 0 there).  Gate weights are one power of two >= 32 per selector row (silu(g) == g in fp32
    from g = 17 on: 1 + exp(-g) rounds to 1), up weights are grid values with 448 among them, the last up column is 0.
    So h[r] = 2^(2p + g) * wu[c(r)] is a grid row with absmax 448 * 2^n, exactly representable in bf16.
    w2 has small grid integers, row I - 1 = 448 * 2^b (h is 0 there).  All sums are small integers: exact in fp32."""
    g = torch.Generator().manual_seed(seed)
    d = sel + 2
    R = sum(sizes)
    x = torch.zeros(R, d)
    p = torch.randint(0, 3, (R,), generator=g)
    c = torch.randint(0, sel, (R,), generator=g)
    x[torch.arange(R), c] = 2.0 ** p.float()
    x[:, sel] = 448.0 * 2.0 ** torch.randint(-2, 3, (R,), generator=g).float()
    w13 = torch.zeros(E, d, 2 * I)
    w2 = torch.zeros(E, I, d_out)
    grid = torch.tensor(_GRID)
    for e in range(E):
        for k in range(sel):
            w13[e, k, :I] = 2.0 ** float(torch.randint(5, 8, (1,), generator=g))          # gate: 32, 64 or 128
            up = grid[torch.randint(0, len(_GRID), (I,), generator=g)]
            up[int(torch.randint(0, I - 1, (1,), generator=g))] = 448.0                  # the row's absmax is 448 * 2^n
            up = up * torch.where(torch.rand(I, generator=g) < 0.5, -1.0, 1.0)
            up[I - 1] = 0.0
            w13[e, k, I:] = up * 2.0 ** float(torch.randint(-3, 1, (1,), generator=g))
        w13[e, sel + 1, :] = 448.0 * 2.0 ** torch.randint(1, 3, (2 * I,), generator=g).float()
        w2[e, :I - 1] = torch.randint(-3, 4, (I - 1, d_out), generator=g).float()
        w2[e, I - 1] = 448.0 * 2.0 ** torch.randint(-3, 0, (d_out,), generator=g).float()
    return x.to(torch.bfloat16), w13.to(torch.bfloat16), w2.to(torch.bfloat16), list(sizes)


def test_identity_quantisation_equals_unquantised_ffn():
    for seed in range(5):
        x, w13, w2, sizes = _on_grid_case(seed=seed)
        # the construction survives the bf16 storage
        q13, s13 = fp8.quantize_weight_channels(w13)
        q2, s2 = fp8.quantize_weight_channels(w2)
        assert torch.equal(fp8.dequantize_weight(q13, s13, torch.float32), w13.float())
        assert torch.equal(fp8.dequantize_weight(q2, s2, torch.float32), w2.float())
        xq, xs = fp8.quantize_rows(x)
        assert torch.equal(fp8.dequantize_rows(xq, xs, torch.float32), x.float())
        out = fp8.moe_experts_forward_fp8(x, q13, s13, q2, s2, sizes)
        ref = ffn.moe_experts_forward(x, w13, w2, sizes)
        assert out.dtype == torch.bfloat16 and out.shape == ref.shape
        assert torch.equal(out, ref), (seed, (out.float() - ref.float()).abs().max())
        assert out.float().abs().max() > 0


def test_intermediate_row_is_quantised_hand_computed():
    # one expert, d = 1, I = 2.  x = 1 -> stored as 448 with scale 1/448.  w13 = [gate 32, gate 32 | up 1, up 0.5625]
    # (each its own channel: exact).  h = [32 * 1, 32 * 0.5625] = [32, 18].  Row scale of h = 32 / 448; 18 / scale = 252;
    # the e4m3 grid around 252 is 240, 256 -> 256; de-quantised 256 * 32 / 448 = 18.2857...  w2 = [[1], [1]]:
    # out = 32 + 18.2857 = 50.2857 -> bf16 (step 0.25) = 50.25.  Without the quantisation of h the answer is 50.0.
    x = torch.tensor([[1.0]], dtype=torch.bfloat16)
    w13 = torch.tensor([[[32.0, 32.0, 1.0, 0.5625]]], dtype=torch.bfloat16)
    w2 = torch.tensor([[[1.0], [1.0]]], dtype=torch.bfloat16)
    q13, s13 = fp8.quantize_weight_channels(w13)
    q2, s2 = fp8.quantize_weight_channels(w2)
    out = fp8.moe_experts_forward_fp8(x, q13, s13, q2, s2, [1])
    assert out.tolist() == [[50.25]]
    assert ffn.moe_experts_forward(x, w13, w2, [1]).tolist() == [[50.0]]
    # a second row with another scale shares nothing with the first: per-row, not per-tensor, scales.
    # x = 4: gate 128, up [4, 2.25] -> h = [512, 288]; 288 / (512 / 448) = 252 -> 256 -> 292.571; out = 804.571 -> bf16
    # (step 4 from 512 on) = 804
    x2 = torch.tensor([[1.0], [4.0]], dtype=torch.bfloat16)
    out2 = fp8.moe_experts_forward_fp8(x2, q13, s13, q2, s2, [2])
    assert out2.tolist() == [[50.25], [804.0]]


def test_weight_scales_are_per_output_channel_hand_computed():
    # two output channels with different magnitudes: w[:, 0] = [448, 100], w[:, 1] = [1.75, 0.4375].
    # channel 0: scale 1, 100 -> grid (96, 104; step 8) -> 96 or 104: 100 is a tie -> even mantissa: 96 = 1.100b * 2^6.
    # channel 1: scale 1.75 / 448 = 2^-8, 0.4375 * 256 = 112 -> on the grid.  A per-tensor scale would flush channel 1.
    w = torch.tensor([[[448.0, 1.75], [100.0, 0.4375]]], dtype=torch.bfloat16)
    q, s = fp8.quantize_weight_channels(w)
    assert s.tolist() == [[1.0, 2.0 ** -8]]
    assert q.shape == (1, 2, 2)                                   # [E, N, K]: K contiguous
    assert q.float().tolist() == [[[448.0, 96.0], [448.0, 112.0]]]
    assert fp8.dequantize_weight(q, s, torch.float32).tolist() == [[[448.0, 1.75], [96.0, 0.4375]]]


def test_zero_rows_and_empty_experts():
    x, w13, w2, _ = _on_grid_case(sizes=(4, 0, 3), seed=7)
    q13, s13 = fp8.quantize_weight_channels(w13)
    q2, s2 = fp8.quantize_weight_channels(w2)
    x[1] = 0                                                     # an all-zero row: scale 1, result 0
    out = fp8.moe_experts_forward_fp8(x, q13, s13, q2, s2, [4, 0, 3])
    assert torch.equal(out[1], torch.zeros_like(out[1]))
    assert torch.equal(out, ffn.moe_experts_forward(x, w13, w2, [4, 0, 3]))
    # the same rows with the sizes moved onto other experts give other results (the sizes pick the weights)
    other = fp8.moe_experts_forward_fp8(x, q13, s13, q2, s2, [0, 7, 0])
    assert torch.equal(other, ffn.moe_experts_forward(x, w13, w2, [0, 7, 0]))
    assert not torch.equal(other, out)
    # no rows at all
    none = fp8.moe_experts_forward_fp8(x[:0], q13, s13, q2, s2, [0, 0, 0])
    assert none.shape == (0, w2.shape[2])


def test_cpu_path_equals_stage_oracles():
    # the cpu_baseline leg computes the function the stage-by-stage oracles define (bf16 storage between its stages:
    # a looser bar than the single-rounding oracle's)
    g = torch.Generator().manual_seed(5)
    T, k, E, d, I = 96, 2, 5, 64, 96
    x = torch.randn(T, d, generator=g).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    ids[ids == 3] = 4                                            # expert 3 gets no rows
    gates = torch.softmax(torch.randn(T, k, generator=g), dim=1)
    w13 = (torch.randn(E, d, 2 * I, generator=g) * 0.1).to(torch.bfloat16)
    w2 = (torch.randn(E, I, d, generator=g) * 0.1).to(torch.bfloat16)
    m, cnt = routing.get_mappings_from_exp_ids(ids, E)
    assert cnt[3] == 0
    ref = ffn.combine(ffn.moe_experts_forward(rows.permute_tokens(x, m), w13, w2, cnt), m, gates)
    timings = {}
    out = cpu_path.expert_layer(x, ids, gates, w13, w2, timings)
    assert out.shape == ref.shape and ffn.max_rel_err(out, ref) <= 2e-2
    assert set(timings) == {"route", "permute", "ffn", "combine", "total"}
    # k = 1 and a single expert: the layer is x @ w1 -> silu * (x @ w3) -> @ w2, scaled by the gate
    one = cpu_path.expert_layer(x[:8], torch.zeros(8, 1, dtype=torch.int32), torch.full((8, 1), 0.5), w13[:1], w2[:1])
    xf = x[:8].float()
    direct = 0.5 * ((torch.nn.functional.silu(xf @ w13[0, :, :I].float()) * (xf @ w13[0, :, I:].float())) @ w2[0].float())
    assert ffn.max_rel_err(one, direct) <= 2e-2
