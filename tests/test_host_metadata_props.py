"""Property tests of the host-side bookkeeping (csrc/meta.hip through ops/metadata.py) on random batches: what the
reference's Metadata methods guarantee by construction (csrc/include/datatypes.hpp:228-247, 343-433) must hold for
every input, and the wire bytes (datatypes.hpp:223-226) must survive a round trip and reject every proper prefix."""
import struct

import numpy as np
import pytest
from hypothesis import given, settings, strategies as st

from disagmoe_amd import _lib
from disagmoe_amd.ops import metadata as md

rows = st.integers(min_value=0, max_value=48)


def _batch(draw, n, experts=8):
    ints = lambda lo, hi: st.lists(st.integers(lo, hi), min_size=n, max_size=n)
    return dict(req_ids=draw(ints(0, 50)), exp_ids=draw(ints(0, experts - 1)), attn_dp_ranks=draw(ints(0, 3)),
                init_prefill_lens=draw(st.lists(st.sampled_from([-1, 0, 5, 17]), min_size=n, max_size=n)),
                topk_weights=draw(st.lists(st.floats(0, 1, width=32), min_size=n, max_size=n)))


@st.composite
def batches(draw):
    n = draw(rows)
    return md.Metadata(shape=[n, 64], dtype="bf16", layer_id=draw(st.integers(0, 63)), **_batch(draw, n))


@settings(max_examples=40, deadline=None)
@given(batches())
def test_sort_by_prefill_order_is_a_stable_ranking(meta):
    n = meta.num_tokens()
    # the reference's comparator: DP rank; prefill rows (length != -1) before decode rows; prefill rows by request id;
    # the decode rows of a rank compare equal
    before = [(r, 0, q) if p != -1 else (r, 1, 0) for r, p, q in zip(meta.attn_dp_ranks, meta.init_prefill_lens, meta.req_ids)]
    keep = dict(req=list(meta.req_ids), w=list(meta.topk_weights))
    mapping = meta.sort_by_prefill_order()
    assert sorted(mapping) == list(range(n))                       # a permutation
    # row i went to mapping[i]; read in the new order the keys ascend, and equal keys keep their old order
    inverse = [0] * n
    for i, m in enumerate(mapping):
        inverse[m] = i
    keys = [before[i] for i in inverse]
    assert keys == sorted(keys)
    for a, b in zip(range(n - 1), range(1, n)):
        if keys[a] == keys[b]:
            assert inverse[a] < inverse[b]
    # every list moved along, the expert ids are dropped (update_exp_ids({}, mapping))
    assert meta.exp_ids == []
    assert [meta.req_ids[mapping[i]] for i in range(n)] == keep["req"]
    assert np.array_equal(np.float32([meta.topk_weights[mapping[i]] for i in range(n)]), np.float32(keep["w"]))


@settings(max_examples=40, deadline=None)
@given(batches(), st.integers(1, 8))
def test_batch_sizes_and_host_mappings_agree(meta, experts):
    ids = [e % experts for e in meta.exp_ids]
    sizes = md.expert_batch_sizes(ids, experts)
    assert sizes == np.bincount(np.asarray(ids, dtype=np.int64), minlength=experts).tolist()
    mappings, cnt = md.host_mappings(ids, experts)
    assert cnt == sizes and sorted(mappings) == list(range(len(ids)))
    # experts ascending along the destination rows; inside an expert the first row takes the last slot
    dest = [0] * len(ids)
    for i, m in enumerate(mappings):
        dest[m] = i
    assert [ids[i] for i in dest] == sorted(ids)
    for e in range(experts):
        src = [i for i in dest if ids[i] == e]
        assert src == sorted(src, reverse=True)
    sel = list(range(experts - 1, -1, -2))
    assert md.expert_batch_sizes(ids, experts, sel) == [sizes[e] for e in sel]


@settings(max_examples=40, deadline=None)
@given(batches())
def test_wire_round_trip_and_prefixes(meta):
    blob = meta.serialize()
    back = md.Metadata.deserialize(blob)
    assert (back.shape, back.dtype, back.layer_id) == (meta.shape, meta.dtype, meta.layer_id)
    assert (back.req_ids, back.exp_ids, back.attn_dp_ranks, back.init_prefill_lens) == \
        (meta.req_ids, meta.exp_ids, meta.attn_dp_ranks, meta.init_prefill_lens)
    assert np.array_equal(np.float32(back.topk_weights), np.float32(meta.topk_weights))
    assert back.serialize() == blob
    # the layout by hand: u64 count of shape, the shape, u64 length of dtype, ...
    assert struct.unpack_from("<Q", blob, 0)[0] == len(meta.shape)
    assert len(blob) == 8 * 7 + 8 * len(meta.shape) + len(meta.dtype) + 4 + 4 * 5 * meta.num_tokens()
    for cut in {0, 1, 7, 8, len(blob) // 2, len(blob) - 1}:
        if cut < len(blob):
            with pytest.raises(_lib.DmoeError):
                md.Metadata.deserialize(blob[:cut])
    with pytest.raises(_lib.DmoeError):
        md.Metadata.deserialize(blob + b"\0")
