"""Row movement parity (bit-exact) and combine parity of the HIP kernels."""
import pytest
import torch

from disagmoe_amd import workloads
from disagmoe_amd.ops import memory
from oracle import ffn, routing, rows
from helpers import TOL_BF16, announce, dev, max_rel_err

pytestmark = pytest.mark.gpu


def test_reference_permute_case():
    # tests/ops/test_memory.py:8-31
    announce(test="permute_reference_case")
    g = torch.Generator().manual_seed(0)
    t = torch.randn(64, 4096, generator=g).to(torch.bfloat16)
    ids = torch.randint(2, 8, (64,), generator=g)
    mappings, cnt = memory.get_mappings_from_exp_ids(ids, 8)
    std = torch.empty_like(t)
    for i in range(64):
        std[mappings[i], :] = t[i, :]
    assert torch.equal(memory.permute_tokens_triton(t.to(dev()), mappings).cpu(), std)
    assert torch.equal(memory.permute_tokens_cuda(t.to(dev()), mappings).cpu(), std)
    assert torch.equal(memory.permute_tokens_cuda(t.to(dev()), torch.tensor(mappings, device=dev())).cpu(), std)


@pytest.mark.parametrize("T,d,k,E", [(1, 8, 1, 1), (5, 8, 2, 3), (37, 1024, 2, 8), (64, 4096, 1, 8), (100, 2048, 6, 64),
                                     (33, 7168, 2, 8), (129, 2056, 3, 5), (256, 16384, 2, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_permute_and_gather(T, d, k, E, dtype):
    announce(test="permute", T=T, d=d, k=k, E=E, dtype=dtype)
    g = torch.Generator().manual_seed(T * 7 + d + k)
    x = torch.randn(T, d, generator=g).to(dtype)
    ids = torch.randint(0, E, (T * k,), generator=g)
    m, _ = routing.get_mappings_from_exp_ids(ids, E)
    ref = rows.permute_tokens(x, m)
    for mt in (torch.int64, torch.int32):
        out = memory.permute_tokens_cuda(x.to(dev()), torch.tensor(m, dtype=mt, device=dev()))
        assert out.dtype == dtype and torch.equal(out.cpu(), ref)
    inv = torch.empty(T * k, dtype=torch.int64)
    inv[torch.tensor(m)] = torch.arange(T * k)
    assert torch.equal(memory.gather_rows(x.to(dev()), (inv // k).to(dev())).cpu(), ref)
    assert torch.equal(memory.gather_rows(x.to(dev()), (inv // k).int().tolist()).cpu(), rows.gather_rows(x, inv // k))


def test_permute_skips_out_of_range_rows_and_gather_zero_fills():
    announce(test="permute_bounds")
    x = torch.arange(4 * 8, dtype=torch.float32).view(4, 8).to(torch.bfloat16).to(dev())
    out = memory.permute_tokens_cuda(x, torch.tensor([2, -1, 0, 7], device=dev()))
    assert torch.equal(out[2], x[0]) and torch.equal(out[0], x[2])
    g = memory.gather_rows(x, torch.tensor([3, 4, -1, 0], device=dev()))
    assert torch.equal(g[0], x[3]) and torch.equal(g[3], x[0]) and g[1].abs().sum() == 0 and g[2].abs().sum() == 0


def test_empty_inputs():
    announce(test="rows_empty")
    x = torch.zeros(0, 64, dtype=torch.bfloat16, device=dev())
    assert memory.permute_tokens_cuda(x, []).shape == (0, 64)
    assert memory.gather_rows(torch.zeros(3, 64, dtype=torch.bfloat16, device=dev()), []).shape == (0, 64)
    w = torch.zeros(0, 2)
    assert memory.combine_tokens(x, [], w).shape == (0, 64)


def test_permute_with_row_scale_matches_torch_statements():
    # engine.py:731-734: output * topk_weights (bf16), then permute_tokens
    announce(test="permute_scale")
    g = torch.Generator().manual_seed(11)
    R, d = 96, 2048
    y = torch.randn(R, d, generator=g).to(torch.bfloat16)
    wts = torch.rand(R, generator=g).to(torch.bfloat16)
    perm = torch.randperm(R, generator=g)
    ref = rows.permute_tokens(y * wts.view(-1, 1), perm)
    out = memory.permute_tokens_cuda(y.to(dev()), perm.to(dev()), row_scale=wts.view(-1, 1).to(dev()))
    assert torch.equal(out.cpu(), ref)


def test_gather_row_ptrs_merges_slabs():
    # TensorBatch::merge (datatypes.hpp:508-549): rows of several slabs land expert-sorted
    announce(test="gather_ptrs")
    g = torch.Generator().manual_seed(12)
    d = 1024
    slabs = [torch.randn(n, d, generator=g).to(torch.bfloat16) for n in (40, 0, 7, 90)]
    ids = [torch.randint(0, 8, (s.shape[0],), generator=g).tolist() for s in slabs]
    m, cnt = routing.merge_by_exp_ids(ids, 8)
    ref = rows.gather_row_slabs(slabs, m)
    dslabs = [s.to(dev()) for s in slabs]
    ptrs = [0] * len(m)
    stream_idx = 0
    for s in dslabs:
        for r in range(s.shape[0]):
            ptrs[m[stream_idx]] = s.data_ptr() + r * d * 2
            stream_idx += 1
    table = torch.tensor(ptrs, dtype=torch.int64, device=dev())
    out = memory.gather_row_ptrs(table, d, torch.bfloat16)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("T,d,k,E", [(1, 8, 1, 1), (9, 16, 2, 4), (200, 1024, 2, 8), (64, 4096, 2, 8), (150, 2048, 6, 64), (31, 7168, 3, 8)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_combine(T, d, k, E, dtype):
    announce(test="combine", T=T, d=d, k=k, E=E, dtype=dtype)
    g = torch.Generator().manual_seed(T + d + k)
    ids = torch.randint(0, E, (T, k), generator=g)
    m, _ = routing.get_mappings_from_exp_ids(ids, E)
    y = torch.randn(T * k, d, generator=g).to(dtype)
    w = torch.softmax(torch.randn(T, k, generator=g), dim=1)
    out = memory.combine_tokens(y.to(dev()), m, w.to(dev()))
    ref = ffn.combine(y, m, w)
    # fp32 accumulation on both sides; fused multiply-add vs separate ops may move the last bit
    assert max_rel_err(out, ref) <= 2 ** -7, max_rel_err(out, ref)
    assert max_rel_err(out, ffn.combine(y, m, w, acc_dtype=torch.float64)) <= TOL_BF16
    # the reference's rounding chain is reproduced bit for bit
    chain = memory.combine_tokens(y.to(dev()), torch.tensor(m, dtype=torch.int32, device=dev()), w.to(dev()), reference_rounding=True)
    assert torch.equal(chain.cpu(), ffn.combine_reference_chain(y, m, w))


def test_permute_then_combine_round_trip():
    announce(test="round_trip")
    g = torch.Generator().manual_seed(5)
    T, d, k, E = 300, 4096, 2, 8
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).to(dev())
    ids = torch.randint(0, E, (T, k), generator=g)
    m, bs, off = memory.route_tokens(ids.to(dev()), E)
    p = memory.permute_tokens_cuda(x, m)
    onehot = torch.zeros(T, k)
    onehot[:, 1] = 1
    assert torch.equal(memory.combine_tokens(p, m, onehot.to(dev())), x)
    half = torch.full((T, k), 0.5)
    assert torch.equal(memory.combine_tokens(p, m, half.to(dev())), x)   # 0.5*x + 0.5*x is exact


@pytest.mark.parametrize("name", ["C2", "C4", "C5"])
def test_full_size_permute_and_combine(name):
    w = workloads.WORKLOADS[name]
    announce(test="rows_full_size", config=name, T=w.T, d=w.d, k=w.k)
    ids, gates = workloads.make_routing(w)
    x = workloads.make_activations(w).to(dev())
    m, bs, off = memory.route_tokens(ids.to(dev()), w.E)
    p = memory.permute_tokens_cuda(x, m)
    # size-independent property: every routed row t sits at mappings[t] (library gather as the checker)
    assert torch.equal(p[m], x.repeat_interleave(w.k, dim=0))
    # rows are expert-sorted: expert id of the row stored at r is non-decreasing
    placed = torch.empty(w.R, dtype=torch.int32, device=dev())
    placed[m] = ids.view(-1).to(dev())
    assert (placed[1:] >= placed[:-1]).all()
    first = torch.zeros(w.T, w.k)
    first[:, 0] = 1
    assert torch.equal(memory.combine_tokens(p, m, first.to(dev())), x)
    if name == "C2":
        assert torch.equal(p.cpu(), rows.permute_tokens(x.cpu(), m.cpu()))
        out = memory.combine_tokens(p, m, gates.to(dev()))
        assert max_rel_err(out, ffn.combine(p.cpu(), m.cpu(), gates)) <= 2 ** -7


def test_row_buffers_beyond_4gib():
    # 640k routed rows of 8 KiB: byte offsets pass 2^32 in the source and the destination of every row kernel
    T, d, k, E = 320000, 4096, 2, 8
    announce(test="rows_beyond_4gib", T=T, d=d, k=k)
    g = torch.Generator(device=dev()).manual_seed(4)
    x = torch.randn(T, d, device=dev(), generator=g, dtype=torch.float32).to(torch.bfloat16)
    ids = torch.randint(0, E, (T, k), device=dev(), generator=g, dtype=torch.int32)
    m, bs, off = memory.route_tokens(ids, E)
    assert int(bs.sum()) == T * k
    p = memory.permute_tokens_cuda(x, m)
    assert p.numel() * 2 > 2 ** 32
    # every routed row t sits at mappings[t]; checked in slabs to bound the checker's memory
    for lo in range(0, T, 80000):
        rows_t = torch.arange(lo * k, (lo + 80000) * k, device=dev())
        assert torch.equal(p[m[rows_t]], x[lo:lo + 80000].repeat_interleave(k, dim=0))
    back = memory.gather_rows(p, m.view(T, k)[:, 1].contiguous())
    assert torch.equal(back, x)
    first = torch.zeros(T, k, device=dev())
    first[:, 0] = 1
    assert torch.equal(memory.combine_tokens(p, m, first), x)


def test_tensor_batch_merge():
    # TensorBatch::merge (csrc/include/datatypes.hpp:508-549): rows of several incoming batches end up sorted by expert
    from disagmoe_amd.ops.metadata import Metadata, TensorBatch
    announce(test="tensor_batch_merge")
    g = torch.Generator().manual_seed(21)
    E, d = 8, 1024
    batches, rows_all, ids_all = [], [], []
    for n in (33, 1, 0, 250, 64):
        ids = torch.randint(0, E, (n,), generator=g).tolist()
        x = torch.randn(n, d, generator=g).to(torch.bfloat16)
        rows_all.append(x)
        ids_all.append(ids)
        batches.append(TensorBatch(x.to(dev()), Metadata(shape=[n, d], req_ids=list(range(n)), exp_ids=ids)))
    merged = TensorBatch.merge(batches, E)
    m_ref, cnt = routing.merge_by_exp_ids(ids_all, E)
    ref = torch.empty(sum(len(i) for i in ids_all), d, dtype=torch.bfloat16)
    ref[torch.tensor(m_ref)] = torch.cat(rows_all)
    assert torch.equal(merged.data.cpu(), ref)
    assert merged.metadata.exp_ids == sorted(v for ids in ids_all for v in ids)
    assert merged.metadata.get_expert_batch_sizes(E) == cnt
