"""Grouped GEMM / expert FFN parity against the fp32-accumulated oracle.

Tolerance (stated by the task): max|out - ref| / max|ref| <= 1e-2 for bf16."""
import pytest
import torch

from disagmoe_amd import workloads
from disagmoe_amd.executor import ExpertsExecutor
from disagmoe_amd.config import ModelConfig
from disagmoe_amd.grouped_gemm import backend as gg
from disagmoe_amd.models.experts import MoEExperts, MoEExpertsSerial
from oracle import ffn
from helpers import TOL_BF16, announce, dev, max_rel_err, ragged_sizes

pytestmark = pytest.mark.gpu


def _rand(shape, seed, std=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)


@pytest.fixture(autouse=True)
def _default_tile():
    gg.set_tile_variant(0)
    yield
    gg.set_tile_variant(0)


def test_reference_gemm_case():
    # tests/ops/test_gemm.py:4-36: E=8, two rows per expert, 1024x1024; gmm == gmm_with_arguments (twice)
    announce(test="gmm_reference_case")
    E, hs = 8, 1024
    w1 = _rand((E, hs, hs), 1).to(dev())
    x = _rand((2 * E, hs), 2).to(dev())
    batch_sizes = torch.tensor([2] * E, dtype=torch.int64)
    y = gg.gmm(x, w1, batch_sizes)
    size, ptr = gg.get_arguments(E, dev())
    workspace = torch.empty([size], dtype=torch.uint8, device=dev())
    y2 = gg.gmm_with_arguments(x, w1, batch_sizes, workspace, ptr)
    y3 = gg.gmm_with_arguments(x, w1, batch_sizes, workspace, ptr)
    assert torch.equal(y, y2) and torch.equal(y, y3)
    assert max_rel_err(y, ffn.gmm(x.cpu(), w1.cpu(), batch_sizes)) <= TOL_BF16


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("E,R,K,N", [(1, 300, 256, 256), (4, 1000, 128, 512), (8, 777, 320, 264), (3, 64, 72, 40),
                                     (5, 1500, 512, 768)])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gmm_ragged(variant, E, R, K, N, trans_b):
    announce(test="gmm_ragged", variant=variant, E=E, R=R, K=K, N=N, trans_b=trans_b)
    gg.set_tile_variant(variant)
    sizes = ragged_sizes(E, R, seed=E * 1000 + R)
    a = _rand((R, K), 3)
    b = _rand((E, N, K) if trans_b else (E, K, N), 4, std=0.05)
    ref = ffn.gmm(a, b, sizes, trans_b=trans_b)
    out = gg.gmm(a.to(dev()), b.to(dev()), sizes.to(dev()), trans_b=trans_b)
    assert out.shape == (R, N) and out.dtype == torch.bfloat16
    assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)


def test_gmm_single_expert_equals_matmul_and_zero_sizes():
    announce(test="gmm_special_cases")
    a = _rand((513, 384), 5).to(dev())
    b = _rand((1, 384, 520), 6, std=0.05).to(dev())
    out = gg.gmm(a, b, torch.tensor([513]))
    assert max_rel_err(out, (a.float() @ b[0].float())) <= TOL_BF16
    # all experts empty: the output buffer is left untouched
    c = torch.full((513, 520), 3.0, dtype=torch.bfloat16, device=dev())
    b4 = _rand((4, 384, 520), 7, std=0.05).to(dev())
    out = gg.gmm(a, b4, torch.zeros(4, dtype=torch.int64), c=c)
    assert out.data_ptr() == c.data_ptr() and (c == 3.0).all()
    # rows past sum(batch_sizes) are left untouched; host or device sizes give the same bits
    c.fill_(3.0)
    sizes = torch.tensor([100, 0, 50, 7])
    gg.gmm(a, b4, sizes, c=c)
    assert (c[157:] == 3.0).all()
    ref = ffn.gmm(a.cpu()[:157], b4.cpu(), sizes)
    assert max_rel_err(c[:157], ref) <= TOL_BF16
    c2 = gg.gmm(a, b4, sizes.to(dev()))
    assert torch.equal(c2[:157], c[:157])
    # sizes that overrun the buffer are clamped, nothing past the last row is touched
    guard = torch.full((600, 520), 5.0, dtype=torch.bfloat16, device=dev())
    gg.gmm(a, b4, torch.tensor([400, 400, 400, 400]), c=guard)
    assert (guard[513:] == 5.0).all()


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("trans_b", [False, True])
def test_gmm_swiglu(variant, trans_b):
    announce(test="gmm_swiglu", variant=variant, trans_b=trans_b)
    gg.set_tile_variant(variant)
    E, R, K, I = 6, 900, 256, 328
    sizes = ragged_sizes(E, R, seed=17)
    a = _rand((R, K), 8)
    w13 = _rand((E, K, 2 * I), 9, std=0.08)
    up = torch.zeros(R, 2 * I)
    o = 0
    for e, n in enumerate(sizes.tolist()):
        up[o:o + n] = a[o:o + n].float() @ w13[e].float()
        o += n
    ref = torch.nn.functional.silu(up[:, :I]) * up[:, I:]
    b = w13.transpose(1, 2).contiguous() if trans_b else w13
    out = gg.gmm_swiglu(a.to(dev()), b.to(dev()), sizes, trans_b=trans_b)
    assert out.shape == (R, I)
    assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)


@pytest.mark.parametrize("E,d,I,R", [(8, 1024, 2816, 1024), (4, 512, 704, 300), (64, 256, 192, 2000)])
def test_moe_experts_forward(E, d, I, R):
    announce(test="moe_experts_forward", E=E, d=d, I=I, R=R)
    layer = MoEExperts(d, I, E, init_std=0.02)
    assert layer.w13_weight.shape == (E, d, 2 * I) and layer.w2_weight.shape == (E, I, d)
    assert sorted(layer.state_dict().keys()) == ["w13_weight", "w2_weight"]
    sizes = ragged_sizes(E, R, seed=E + R)
    x = _rand((R, d), 10).to(dev())
    out = layer.forward(R, x, sizes.to(dev()))
    ref = ffn.moe_experts_forward(x.cpu(), layer.w13_weight.cpu(), layer.w2_weight.cpu(), sizes)
    assert out.shape == (R, d)
    assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)
    # the reference's unfused schedule (four roundings), against the oracle that rounds at the same four places
    chain = ffn.moe_experts_forward_reference_rounding(x.cpu(), layer.w13_weight.cpu(), layer.w2_weight.cpu(), sizes)
    assert max_rel_err(layer.forward_unfused(R, x, sizes.to(dev())), chain) <= TOL_BF16
    # static-buffer path (bs below max_batch_size) gives the same bits as the allocating path
    small = MoEExperts(d, I, E, init_std=0.02, max_batch_size=R)
    small.load_state_dict(layer.state_dict())
    assert torch.equal(small.forward(R, x, sizes.to(dev())), out)


def test_serial_experts_and_executor():
    announce(test="serial_and_executor")
    E, d, I, R = 4, 512, 768, 200
    cfg = ModelConfig(hidden_size=d, num_layers=2, num_heads=8, num_kv_heads=8, num_experts=E, intermediate_size=I,
                      layer_ids=[3, 7], top_k=2, max_batch_size_expert=64)
    ex = ExpertsExecutor(cfg, init_std=0.02)
    assert len(ex.operators) == 2 and isinstance(ex.operators[0], MoEExperts)
    sizes = ragged_sizes(E, R, seed=1)
    x = _rand((R, d), 11).to(dev())
    out = ex.execute(7, R, x, sizes.to(dev()))
    op = ex.operators[1]
    ref = ffn.moe_experts_forward(x.cpu(), op.w13_weight.cpu(), op.w2_weight.cpu(), sizes)
    assert max_rel_err(out, ref) <= TOL_BF16
    serial = MoEExpertsSerial(d, I, E, init_std=0.02)
    serial.load_state_dict(op.state_dict())
    assert max_rel_err(serial.forward(R, x, sizes), ref) <= TOL_BF16
    cfg.enable_grouped_gemm = False
    assert isinstance(ExpertsExecutor(cfg, init_std=0.02).operators[0], MoEExpertsSerial)


@pytest.mark.parametrize("trans_b", [False, True])
def test_gmm_expert_count_limit(trans_b):
    # the tile tables of E + 1 entries live in LDS: up to 1024 experts per call, most of them empty here
    announce(test="gmm_max_experts", trans_b=trans_b)
    from disagmoe_amd._lib import DmoeError
    E, R, K, N = 1024, 700, 128, 256
    g = torch.Generator().manual_seed(3)
    sizes = torch.zeros(E, dtype=torch.int64)
    picks = torch.randperm(E, generator=g)[:40]
    sizes[picks] = torch.randint(1, 30, (40,), generator=g)
    sizes[picks[0]] += R - int(sizes.sum())
    assert int(sizes.sum()) == R and int(sizes.min()) == 0
    a = _rand((R, K), 21)
    b = _rand((E, N, K) if trans_b else (E, K, N), 22, std=0.05)
    out = gg.gmm(a.to(dev()), b.to(dev()), sizes.to(dev()), trans_b=trans_b)
    assert max_rel_err(out, ffn.gmm(a, b, sizes, trans_b=trans_b)) <= TOL_BF16
    with pytest.raises(DmoeError):
        gg.gmm(a.to(dev()), _rand((1025, K, 8), 23).to(dev()), torch.zeros(1025, dtype=torch.int64), trans_b=False)


@pytest.mark.parametrize("trans_b", [False, True])
def test_gmm_weights_beyond_32bit_offsets(trans_b):
    # one expert's weights of 2^32 bytes and more leave the kernel with 32-bit offsets inside an expert; columns at
    # both ends and around the 2^31 / 2^32 byte marks are compared with the oracle
    announce(test="gmm_4gib_expert", trans_b=trans_b)
    E, R, K, N = 2, 96, 16384, 131072 + 256
    g = torch.Generator(device=dev()).manual_seed(9)
    b = torch.empty((E, N, K) if trans_b else (E, K, N), dtype=torch.bfloat16, device=dev())
    for e in range(E):
        b[e].copy_(torch.randn(b.shape[1:], device=dev(), generator=g, dtype=torch.float32).mul_(0.02))
    a = _rand((R, K), 31)
    sizes = torch.tensor([40, 56])
    out = gg.gmm(a.to(dev()), b, sizes, trans_b=trans_b)
    assert out.shape == (R, N)
    cols = torch.cat([torch.arange(0, 64), torch.arange(65536 - 32, 65536 + 32), torch.arange(131072 - 32, 131072 + 32),
                      torch.arange(N - 64, N)])
    b_cols = (b[:, cols, :].transpose(1, 2) if trans_b else b[:, :, cols]).contiguous().cpu()
    ref = ffn.gmm(a, b_cols, sizes)
    assert max_rel_err(out[:, cols.to(dev())], ref) <= TOL_BF16
    assert torch.isfinite(out.float()).all()


@pytest.mark.parametrize("trans_b", [False, True])
@pytest.mark.parametrize("K", [2048, 96])
def test_gmm_decode_sized_batch_on_tall_tiles(trans_b, K):
    # 256-row tiles that are less than half full on average: tiles of at most 112 rows run one phase per stage with
    # reads of their valid row fragments only, the taller ones of the same launch (113, 130 rows: the lower half of the
    # wavefronts has rows too) keep the two alternating phases; an empty expert between them
    announce(test="gmm_decode_tall_tiles", trans_b=trans_b, K=K)
    gg.set_tile_variant(7)
    sizes = torch.tensor([5, 40, 100, 112, 113, 130, 0, 60], dtype=torch.int64)
    E, R, N = len(sizes), int(sizes.sum()), 1024
    a = _rand((R, K), 71)
    b = _rand((E, K, N), 72, std=0.05)
    w13 = _rand((E, K, 2 * N), 73, std=0.05)
    up = ffn.gmm(a, w13, sizes, out_dtype=torch.float32)
    ref_h = torch.nn.functional.silu(up[:, :N]) * up[:, N:]
    bd = b.transpose(1, 2).contiguous() if trans_b else b
    wd = w13.transpose(1, 2).contiguous() if trans_b else w13
    out = gg.gmm(a.to(dev()), bd.to(dev()), sizes, trans_b=trans_b)
    assert max_rel_err(out, ffn.gmm(a, b, sizes)) <= TOL_BF16
    h = gg.gmm_swiglu(a.to(dev()), wd.to(dev()), sizes, trans_b=trans_b)
    assert max_rel_err(h, ref_h) <= TOL_BF16


@pytest.mark.parametrize("variant", [0, 5, 6, 7, 8])
@pytest.mark.parametrize("K", [32, 64, 96])
def test_gmm_few_stages(variant, K):
    # one, two and three 32-k stages: fewer than the LDS pipeline is deep (its prologue, tail and the staging of the
    # results in a free stage buffer all take their short paths)
    announce(test="gmm_few_stages", variant=variant, K=K)
    gg.set_tile_variant(variant)
    E, R, N = 3, 700, 512
    sizes = ragged_sizes(E, R, seed=K)
    a = _rand((R, K), 41)
    b = _rand((E, K, N), 42, std=0.1)
    out = gg.gmm(a.to(dev()), b.to(dev()), sizes)
    assert max_rel_err(out, ffn.gmm(a, b, sizes)) <= TOL_BF16
    w13 = _rand((E, K, 2 * N), 43, std=0.1)
    up = ffn.gmm(a, w13, sizes, out_dtype=torch.float32)
    ref = torch.nn.functional.silu(up[:, :N]) * up[:, N:]
    assert max_rel_err(gg.gmm_swiglu(a.to(dev()), w13.to(dev()), sizes), ref) <= TOL_BF16


def _split_case(E, R, K, N, seed, swiglu, trans_b):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(R, K, generator=g).to(torch.bfloat16)
    cols = 2 * N if swiglu else N
    b = (torch.randn(E, K, cols, generator=g) * 0.05).to(torch.bfloat16)
    sizes = ragged_sizes(E, R, seed=seed, empty_every=0)
    if swiglu:
        u = ffn.gmm(a, b, sizes, out_dtype=torch.float32)
        ref = (torch.nn.functional.silu(u[:, :N]) * u[:, N:]).to(torch.bfloat16)
    else:
        ref = ffn.gmm(a, b, sizes)
    if trans_b:
        b = b.transpose(1, 2).contiguous()
    return a.to(dev()), b.to(dev()), sizes.to(dev()), ref


def _expected_split(sizes, n_out, swiglu, K, workspace_bytes, fp8=False):
    """Pieces per tile of the last round (1: nothing is cut) and the tile rows, as the library itself plans the launch
    (dmoe_gmm_plan, which runs the code the launch runs)."""
    plan = gg.launch_plan(int(sum(sizes)), len(sizes), K, n_out, swiglu=swiglu, fp8=fp8, workspace_bytes=workspace_bytes,
                          batch_sizes=sizes)
    return plan["pieces_per_cut_tile"], plan["tile_rows"]


@pytest.mark.parametrize("variant", [5, 6, 7, 8, 0])
@pytest.mark.parametrize("swiglu,trans_b", [(False, False), (True, False), (False, True), (True, True)])
@pytest.mark.parametrize("E,R,K,N", [(2, 200, 8192, 256), (3, 700, 8192, 512), (2, 150, 16384, 256), (8, 1500, 1024, 768)])
def test_gmm_tail_tiles_cut_along_k(variant, swiglu, trans_b, E, R, K, N):
    # fewer tiles than a whole number of rounds and a long K: the tiles of the last round are cut in pieces whose fp32
    # partial sums meet in the workspace.  Against the oracle, bit-reproducible call after call, the state block left
    # zeroed, and the same bits from gmm() (the module's own pair of the same size) and gmm_with_arguments().
    announce(test="gmm_split_tail", variant=variant, swiglu=swiglu, trans_b=trans_b, E=E, R=R, K=K, N=N)
    gg.set_tile_variant(variant)
    a, b, sizes, ref = _split_case(E, R, K, N, seed=E + R + K, swiglu=swiglu, trans_b=trans_b)
    fn = gg.gmm_swiglu if swiglu else gg.gmm
    size, ptr = gg.get_arguments(E, dev())
    workspace = torch.full([size], 0xA5, dtype=torch.uint8, device=dev())        # any contents
    outs = [fn(a, b, sizes, trans_b=trans_b, workspace=workspace, arguments_ptr=ptr) for _ in range(3)]
    torch.cuda.synchronize()
    assert max_rel_err(outs[0], ref) <= TOL_BF16, max_rel_err(outs[0], ref)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    assert int(gg._STATE_BLOCKS[ptr].count_nonzero()) == 0
    assert torch.equal(fn(a, b, sizes, trans_b=trans_b), outs[0])
    # pieces were written where the plan cuts tiles (the head of the workspace no longer holds the fill pattern), and
    # only there; the cases are chosen so that every forced tile height cuts at least once
    split, tile_rows = _expected_split(sizes.cpu().tolist(), N, swiglu, K, size)
    print(f"[split] tile rows {tile_rows}: {split} pieces per tile of the last round")
    assert variant not in (5, 6, 7, 8) or tile_rows == {5: 64, 6: 128, 7: 256, 8: 256}[variant]
    assert bool((workspace[:4096] == 0xA5).all()) == (split == 1)
    # without a workspace nothing is cut: the same product summed in one piece
    whole = fn(a, b, sizes, trans_b=trans_b, arguments_ptr=ptr)
    assert max_rel_err(whole, ref) <= TOL_BF16
    assert max_rel_err(whole, outs[0].cpu()) <= 2e-2


@pytest.mark.parametrize("variant", [5, 6, 7, 8])
@pytest.mark.parametrize("swiglu", [False, True])
def test_cut_launches_alternating_operands_on_one_state(variant, swiglu):
    # Two different problems A, B, A, B, ... through cut launches that share one state block and one workspace: a
    # partial sum or an arrival count left over from the launch before (or a stale copy of it in some cache) would
    # show, because the launch before had other operands.  Every result against the oracle and against the same
    # launch without a workspace (nothing cut).
    announce(test="gmm_split_alternating", variant=variant, swiglu=swiglu)
    gg.set_tile_variant(variant)
    E, K, N = 3, 8192, 512
    cases = [_split_case(E, 700, K, N, seed=11, swiglu=swiglu, trans_b=False),
             _split_case(E, 640, K, N, seed=12, swiglu=swiglu, trans_b=False)]
    fn = gg.gmm_swiglu if swiglu else gg.gmm
    size, ptr = gg.get_arguments(E, dev())
    workspace = torch.empty([size], dtype=torch.uint8, device=dev())
    for a, b, sizes, _ in cases:
        split, _rows = _expected_split(sizes.cpu().tolist(), N, swiglu, K, size)
        assert split > 1
    uncut = [fn(a, b, sizes, arguments_ptr=ptr) for a, b, sizes, _ in cases]
    outs = []
    for rep in range(6):
        a, b, sizes, _ = cases[rep % 2]
        outs.append(fn(a, b, sizes, workspace=workspace, arguments_ptr=ptr))     # back to back, no synchronisation
    torch.cuda.synchronize()
    for rep, out in enumerate(outs):
        ref = cases[rep % 2][3]
        assert max_rel_err(out, ref) <= TOL_BF16, (rep, max_rel_err(out, ref))
        assert max_rel_err(out, uncut[rep % 2].cpu()) <= 2e-2, rep
        assert torch.equal(out, outs[rep % 2]), rep
    assert int(gg._STATE_BLOCKS[ptr].count_nonzero()) == 0
    gg.set_tile_variant(0)


@pytest.mark.parametrize("T,k,E,K,I", [(300, 2, 8, 256, 384), (1000, 1, 3, 1024, 128), (512, 6, 64, 512, 256),
                                        (64, 2, 8, 8192, 256), (2048, 2, 4, 96, 136)])
def test_gmm_swiglu_rows_equals_permute_then_gmm(T, k, E, K, I):
    # The gate-up projection that fetches the tokens' rows by their place in the expert-sorted order against the pair
    # it replaces (permute, then the same kernel on the copy): the same bits, and the oracle's values.  Experts without
    # rows, experts of a few rows, a long K whose tiles are cut in pieces (one state block and workspace for both).
    from disagmoe_amd.ops import memory
    announce(test="gmm_swiglu_rows", T=T, k=k, E=E, K=K, I=I)
    g = torch.Generator().manual_seed(T + K)
    x = torch.randn(T, K, generator=g).to(torch.bfloat16)
    w13 = (torch.randn(E, K, 2 * I, generator=g) * 0.05).to(torch.bfloat16)
    ids = torch.stack([torch.randperm(E, generator=g)[:k] for _ in range(T)]).to(torch.int32)
    if E > 2:
        ids[ids == 1] = 2 if k == 1 else ids[ids == 1]                # (top-1: an expert without rows)
    m, bs, off, row_token = memory.route_tokens_with_sources(ids.to(dev()), E)
    assert torch.equal(row_token.cpu().long(), torch.argsort(m.cpu()) // k)
    m0, bs0, off0 = memory.route_tokens(ids.to(dev()), E)
    assert torch.equal(m, m0) and torch.equal(bs, bs0) and torch.equal(off, off0)
    xp = memory.permute_tokens_cuda(x.to(dev()), m)
    size, ptr = gg.get_arguments(E, dev())
    workspace = torch.empty([size], dtype=torch.uint8, device=dev())
    gg.set_tile_variant(7)                                            # the kernel that the row-fetching form runs on
    want = gg.gmm_swiglu(xp, w13.to(dev()), bs, workspace=workspace, arguments_ptr=ptr)
    gg.set_tile_variant(0)
    got = gg.gmm_swiglu_rows(x.to(dev()), row_token, w13.to(dev()), bs, workspace=workspace, arguments_ptr=ptr)
    again = gg.gmm_swiglu_rows(x.to(dev()), row_token, w13.to(dev()), bs, workspace=workspace, arguments_ptr=ptr)
    torch.cuda.synchronize()
    assert torch.equal(got, want) and torch.equal(again, want)
    u = ffn.gmm(xp.cpu(), w13, bs.cpu(), out_dtype=torch.float32)
    ref = (torch.nn.functional.silu(u[:, :I]) * u[:, I:]).to(torch.bfloat16)
    assert max_rel_err(got, ref) <= TOL_BF16
    assert int(gg._STATE_BLOCKS[ptr].count_nonzero()) == 0


@pytest.mark.parametrize("swiglu", [False, True])
@pytest.mark.parametrize("sizes", [[700] + [0] * 40 + [324] + [0] * 22,          # two experts hold everything
                                   [40, 1, 0, 300, 0, 0, 7, 676],                  # skewed, 8 experts
                                   [16] * 64])                                     # even: the estimate is right already
def test_batch_sizes_on_the_host_shape_the_launch(sizes, swiglu):
    """``batch_sizes`` as a host tensor (what the reference passes off its CUTLASS path, engine.py:377-380,690-701), or a
    host copy beside the device tensor: the library counts the tiles instead of estimating them from rows / E.  Same
    results as with device sizes only (to the tolerance: another tile height may cut another tail along K), the plan it
    reports is the exact one, and host sizes that disagree with the device's cost nothing but speed."""
    announce(test="gmm_host_sizes", sizes=sizes[:8], E=len(sizes), swiglu=swiglu)
    E, K, N = len(sizes), 512, 768
    R = sum(sizes)
    bs = torch.tensor(sizes, dtype=torch.int64)
    a = _rand((R, K), 31)
    b = _rand((E, K, 2 * N if swiglu else N), 32, std=0.05)
    ref = ffn.gmm(a, b, bs, out_dtype=torch.float32)
    if swiglu:
        ref = torch.nn.functional.silu(ref[:, :N]) * ref[:, N:]
    run = gg.gmm_swiglu if swiglu else gg.gmm
    a_d, b_d = a.to(dev()), b.to(dev())
    out_dev = run(a_d, b_d, bs.to(dev()))
    out_host = run(a_d, b_d, bs)                                          # a host tensor, as the reference passes it
    out_both = run(a_d, b_d, bs.to(dev()), host_batch_sizes=bs)
    wrong = torch.tensor(sizes[::-1], dtype=torch.int64)
    out_wrong = run(a_d, b_d, bs.to(dev()), host_batch_sizes=wrong)       # the kernels read the device's sizes
    for out in (out_dev, out_host, out_both, out_wrong):
        assert max_rel_err(out, ref) <= TOL_BF16, max_rel_err(out, ref)
    assert torch.equal(out_host, out_both)
    est = gg.launch_plan(R, E, K, N, swiglu=swiglu, batch_sizes=bs)
    exact = gg.launch_plan(R, E, K, N, swiglu=swiglu, batch_sizes=bs, sizes_passed=True)
    n_tiles = -(-N // (128 if swiglu else 256))
    for plan in (est, exact):
        assert plan["tiles"] == sum(-(-n // plan["tile_rows"]) for n in sizes) * n_tiles, plan
    # without the sizes the grid is sized for rows / tile_rows + E m-tiles, with them for the tiles there are
    print(f"[plan] estimated {est['tile_rows']} rows x {est['workgroups']} workgroups, exact {exact['tile_rows']} x {exact['workgroups']}")
    assert exact["workgroups"] <= est["workgroups"] or exact["tile_rows"] != est["tile_rows"], (est, exact)
    assert exact["workgroups"] <= -(-exact["tiles"] // 8) * 8, exact


def test_gmm_launches_on_two_streams_keep_their_own_state():
    # a recorded graph of a layer (its own state block and workspace) is replayed on one stream while 80 eager launches
    # with the module-wide pair of another stream run beside it; both give the bits of their serial runs
    announce(test="gmm_two_streams")
    E, R, K, N = 8, 2000, 1024, 1536
    a, b, sizes, ref = _split_case(E, R, K, N, seed=5, swiglu=False, trans_b=False)
    a2, b2, sizes2, ref2 = _split_case(E, 1800, 2048, 1024, seed=6, swiglu=True, trans_b=False)
    size, ptr = gg.get_arguments(E, dev())
    workspace = torch.empty([size], dtype=torch.uint8, device=dev())
    serial = gg.gmm(a, b, sizes, workspace=workspace, arguments_ptr=ptr).clone()
    serial2 = gg.gmm_swiglu(a2, b2, sizes2).clone()
    assert max_rel_err(serial, ref) <= TOL_BF16 and max_rel_err(serial2, ref2) <= TOL_BF16
    out = torch.empty_like(serial)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        gg.gmm(a, b, sizes, c=out, workspace=workspace, arguments_ptr=ptr)
    # a launch without a caller-owned state block cannot be recorded
    from disagmoe_amd._lib import DmoeError
    with pytest.raises(DmoeError):
        with torch.cuda.graph(torch.cuda.CUDAGraph(), stream=side):
            from disagmoe_amd import _lib
            _lib.call("dmoe_gmm", a.data_ptr(), b.data_ptr(), out.data_ptr(), sizes.data_ptr(), R, E, K, N, 0, _lib.BF16,
                      None, None, 0, None, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    eager = []
    for round_ in range(4):
        out.zero_()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for _ in range(5):
                graph.replay()
        eager = [gg.gmm_swiglu(a2, b2, sizes2) for _ in range(20)]     # the default stream's pair
        torch.cuda.synchronize()
        assert torch.equal(out, serial), round_
        assert all(torch.equal(e, serial2) for e in eager), round_
