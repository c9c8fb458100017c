"""Per-row bookkeeping of the expert worker (host code in the C++ library) against the oracle and the
reference's own known answer.  No device work: these run without a GPU."""
import json
import os

import numpy as np
import pytest

from disagmoe_amd import _lib
from disagmoe_amd.ops import metadata
from disagmoe_amd.ops.metadata import Metadata
from oracle import routing


def _load(golden_dir, name):
    with open(os.path.join(golden_dir, name)) as f:
        return json.load(f)


def test_prefill_order_reference_known_answer(golden_dir):
    # tests/engine/test_exp_engine.py:29-40 of the reference: lens [0,-1,0,-1,-1,0,0] read [0,0,0,0,-1,-1,-1] afterwards
    kat = _load(golden_dir, "prefill_kat.json")
    mapping = metadata.sort_by_prefill_order(kat["req_ids"], kat["attn_dp_ranks"], kat["init_prefill_lens"])
    assert mapping == kat["mapping"]
    assert metadata.move_row_infos(kat["init_prefill_lens"], mapping) == kat["sorted_init_prefill_lens"]
    meta = Metadata(shape=[7, 4096], req_ids=list(kat["req_ids"]), exp_ids=[0] * 7,
                    init_prefill_lens=list(kat["init_prefill_lens"]))
    assert meta.sort_by_prefill_order() == kat["mapping"]
    assert meta.init_prefill_lens == kat["sorted_init_prefill_lens"]
    assert meta.req_ids == [0, 2, 5, 6, 1, 3, 4] and meta.exp_ids == []


@pytest.mark.parametrize("n,ranks,seed", [(1, 1, 0), (2, 1, 1), (64, 1, 2), (257, 3, 3), (5000, 4, 4), (49152, 8, 5)])
def test_prefill_order_matches_oracle(n, ranks, seed):
    rng = np.random.default_rng(seed)
    req = rng.integers(0, max(2, n // 3), n).tolist()          # repeated request ids: ties among prefill rows
    dp = rng.integers(0, ranks, n).tolist()
    lens = np.where(rng.random(n) < 0.4, -1, rng.integers(0, 100, n)).tolist()
    mapping = metadata.sort_by_prefill_order(req, dp, lens)
    assert mapping == routing.sort_by_prefill_order(req, dp, lens)
    # properties that do not depend on the oracle: a permutation; sorted by (rank, decode?, request id of prefill rows)
    assert sorted(mapping) == list(range(n))
    inv = np.argsort(np.asarray(mapping))
    key = [(dp[i], lens[i] == -1, req[i] if lens[i] != -1 else 0) for i in inv]
    assert key == sorted(key)
    # rows that compare equal keep their order
    for a, b in zip(inv[:-1], inv[1:]):
        ka = (dp[a], lens[a] == -1, req[a] if lens[a] != -1 else 0)
        kb = (dp[b], lens[b] == -1, req[b] if lens[b] != -1 else 0)
        assert ka != kb or a < b


def test_prefill_order_empty():
    assert metadata.sort_by_prefill_order([], [], []) == []


@pytest.mark.parametrize("n", [0, 1, 17, 1000])
def test_move_row_infos(n):
    rng = np.random.default_rng(n)
    mapping = rng.permutation(n).tolist()
    ints = rng.integers(-5, 1000, n).tolist()
    floats = rng.random(n).astype(np.float32).tolist()
    assert metadata.move_row_infos(ints, mapping) == routing.apply_row_mapping(ints, mapping)
    assert metadata.move_row_infos(floats, mapping, dtype=np.float32) == routing.apply_row_mapping(floats, mapping)
    wide = rng.integers(-2**40, 2**40, n).tolist()
    assert metadata.move_row_infos(wide, mapping, dtype=np.int64) == routing.apply_row_mapping(wide, mapping)


def test_move_row_infos_rejects_bad_mapping():
    with pytest.raises(_lib.DmoeError):
        metadata.move_row_infos([1, 2, 3], [0, 1, 3])
    with pytest.raises(_lib.DmoeError):
        metadata.move_row_infos([1, 2, 3], [0, -1, 2])


@pytest.mark.parametrize("n,E", [(0, 4), (7, 2), (1000, 8), (49152, 64)])
def test_expert_batch_sizes(n, E):
    rng = np.random.default_rng(n + E)
    ids = rng.integers(0, E, n).tolist()
    assert metadata.expert_batch_sizes(ids, E) == np.bincount(np.asarray(ids, dtype=np.int64), minlength=E).tolist()
    assert metadata.expert_batch_sizes(ids, E) == routing.expert_batch_sizes(ids, E).tolist()
    inner = [E - 1, 0] + ([E // 2] if E > 2 else [])
    assert metadata.expert_batch_sizes(ids, E, inner) == routing.expert_batch_sizes(ids, E, inner).tolist()
    with pytest.raises(_lib.DmoeError):
        metadata.expert_batch_sizes([0, E], E)
    with pytest.raises(_lib.DmoeError):
        metadata.expert_batch_sizes(ids, E, [E])


def test_metadata_topk_and_update():
    meta = Metadata(shape=[3, 8], req_ids=[10, 11, 12], init_prefill_lens=[5, -1, 7], attn_dp_ranks=[0, 1, 0])
    meta.duplicate_topk(2)
    # k-major: copy j of request i at j * n + i (datatypes.hpp:364-370)
    assert meta.req_ids == [10, 11, 12, 10, 11, 12] and meta.shape == [6, 8]
    assert meta.init_prefill_lens == [5, -1, 7, 5, -1, 7] and meta.attn_dp_ranks == [0, 1, 0, 0, 1, 0]
    meta.topk_weights = [0.5, 0.25, 0.125, 1.0, 2.0, 4.0]
    mapping = [5, 1, 4, 2, 0, 3]
    meta.update_exp_ids([2, 0, 2, 1, 0, 2], mapping)
    assert meta.exp_ids == routing.apply_row_mapping([2, 0, 2, 1, 0, 2], mapping) == [0, 0, 1, 2, 2, 2]
    assert meta.req_ids == routing.apply_row_mapping([10, 11, 12, 10, 11, 12], mapping)
    assert meta.topk_weights == routing.apply_row_mapping([0.5, 0.25, 0.125, 1.0, 2.0, 4.0], mapping)
    assert meta.get_expert_batch_sizes(3) == [2, 1, 3]
    meta.shrink_topk(2)
    assert meta.shape == [3, 8] and len(meta.req_ids) == 6      # only the row count shrinks (datatypes.hpp:349-352)
    meta.step_layer()
    assert meta.layer_id == 1
    one = Metadata(shape=[2, 8], req_ids=[1, 2])
    one.duplicate_topk(1)
    one.shrink_topk(1)
    assert one.shape == [2, 8] and one.req_ids == [1, 2]


def test_host_mappings_known_answers_and_oracle(golden_dir):
    for case in _load(golden_dir, "routing_kat.json")["cases"]:
        m, cnt = metadata.host_mappings(case["ids"], case["E"])
        assert m == case["mappings"] and cnt == case["exp_cnt"]
    for n, E, seed in [(0, 3, 0), (1, 1, 1), (1000, 8, 2), (49152, 64, 3), (300, 100, 4)]:   # more than the reference's 32 experts
        ids = np.random.default_rng(seed).integers(0, E, n).tolist()
        m, cnt = metadata.host_mappings(ids, E)
        m_ref, cnt_ref = routing.get_mappings_from_exp_ids(ids, E)
        assert m == m_ref and cnt == cnt_ref
    with pytest.raises(_lib.DmoeError):
        metadata.host_mappings([0, 5], 5)


def test_merge_by_exp_ids_matches_oracle():
    rng = np.random.default_rng(12)
    E = 6
    metas, batches = [], []
    base = 0
    for n in (5, 0, 17, 9):
        ids = rng.integers(0, E, n).tolist()
        batches.append(ids)
        metas.append(Metadata(shape=[n, 64], layer_id=3, req_ids=list(range(base, base + n)), exp_ids=ids,
                              attn_dp_ranks=rng.integers(0, 2, n).tolist(), init_prefill_lens=rng.integers(-1, 9, n).tolist(),
                              topk_weights=rng.random(n).astype(np.float32).tolist() if n != 9 else []))
        base += n
    merged, mappings = Metadata.merge_by_exp_ids(metas, E)
    m_ref, cnt_ref = routing.merge_by_exp_ids(batches, E)
    assert mappings == m_ref
    cat = lambda name: [v for m in metas for v in getattr(m, name)]
    assert merged.shape == [31, 64] and merged.layer_id == 3
    assert merged.exp_ids == routing.apply_row_mapping(cat("exp_ids"), mappings) == sorted(cat("exp_ids"))
    assert merged.req_ids == routing.apply_row_mapping(cat("req_ids"), mappings)
    assert merged.attn_dp_ranks == routing.apply_row_mapping(cat("attn_dp_ranks"), mappings)
    assert merged.init_prefill_lens == routing.apply_row_mapping(cat("init_prefill_lens"), mappings)
    weights = cat("topk_weights") + [0.0] * 9      # the last batch came without weights
    assert merged.topk_weights == routing.apply_row_mapping(weights, mappings)
    assert merged.get_expert_batch_sizes(E) == cnt_ref


def test_wire_format_golden_blobs(golden_dir):
    # byte-exact writer and reader against hand-assembled blobs (cereal binary archive, field order of
    # Metadata::serialize, datatypes.hpp:223-226)
    import json
    import os
    from disagmoe_amd.ops.metadata import Metadata
    from disagmoe_amd._lib import DmoeError
    for case in json.load(open(os.path.join(golden_dir, "metadata_wire.json"))):
        blob = bytes.fromhex(case["hex"].replace(" ", ""))
        meta = Metadata(**case["fields"])
        assert meta.serialize() == blob
        back = Metadata.deserialize(blob)
        for name, value in case["fields"].items():
            assert getattr(back, name) == value, name
        assert back.serialize() == blob
        # a blob cut short or with bytes left over is refused
        for bad in (blob[:-1], blob + b"\0", blob[:13]):
            with pytest.raises(DmoeError):
                Metadata.deserialize(bad)
    # a count that points past the end of the blob
    with pytest.raises(DmoeError):
        Metadata.deserialize((2 ** 40).to_bytes(8, "little") + b"\0" * 64)


def test_wire_format_round_trip_after_the_expert_step():
    from disagmoe_amd.ops.metadata import Metadata
    rng = np.random.default_rng(3)
    n = 257
    meta = Metadata(shape=[n, 4096], layer_id=7, req_ids=rng.integers(0, 10 ** 6, n).tolist(),
                    exp_ids=rng.integers(0, 64, n).tolist(), attn_dp_ranks=rng.integers(0, 4, n).tolist(),
                    init_prefill_lens=rng.choice([-1, 5, 900], n).tolist(), topk_weights=rng.random(n, dtype=np.float32).tolist())
    blob = meta.serialize()
    assert len(blob) == 8 * 3 + (8 + 4) + 4 + 5 * 8 + 5 * 4 * n
    back = Metadata.deserialize(blob)
    assert back == meta
    back.sort_by_prefill_order()
    again = Metadata.deserialize(back.serialize())
    assert again == back and again.exp_ids == []
