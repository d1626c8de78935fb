"""Shape inference of the connector side, against the 12 cases of the
reference's python/tests/test_worker_kv_layout.py (held as data in
tests/golden/reference_kats.json)."""

import pytest

from pegaflow_amd import infer_kv_cache_registration, resolve_transfer_backend


class FakeTensor:
    def __init__(self, shape, stride, element_size=2):
        self.shape = tuple(shape)
        self._stride = tuple(stride)
        self._element_size = element_size

    def stride(self):
        return self._stride

    def element_size(self):
        return self._element_size


def test_kv_registration_kats(kats):
    assert len(kats["kv_registration"]) == 12
    for case in kats["kv_registration"]:
        shape, stride, esz = case["tensor"]
        kwargs = {"is_mla": case.get("is_mla", False),
                  "is_recurrent_state": case.get("is_recurrent_state", False)}
        exp = case["expect"]
        if "error_match" in exp:
            with pytest.raises(ValueError, match=exp["error_match"]):
                infer_kv_cache_registration(FakeTensor(shape, stride, esz),
                                            case["logical_block_size"], **kwargs)
            continue
        info = infer_kv_cache_registration(FakeTensor(shape, stride, esz),
                                           case["logical_block_size"], **kwargs)
        for key, val in exp.items():
            assert getattr(info, key) == val, (case["name"], key)


def test_baseline_config_shapes():
    """The registration each BASELINE config's tensor produces."""
    def contiguous(shape):
        stride, acc = [], 1
        for d in reversed(shape):
            stride.append(acc)
            acc *= d
        return FakeTensor(shape, list(reversed(stride)), 2)

    llama = infer_kv_cache_registration(contiguous([2, 8192, 16, 8, 128]), 16)
    assert (llama.layout, llama.num_blocks, llama.bytes_per_block, llama.kv_stride_bytes,
            llama.segments) == ("KV-first", 8192, 32768, 268435456, 2)
    mla = infer_kv_cache_registration(contiguous([4096, 64, 576]), 64, is_mla=True)
    assert (mla.layout, mla.num_blocks, mla.bytes_per_block, mla.segments) == \
        ("blocks-first", 4096, 73728, 1)


def test_resolve_transfer_backend():
    assert resolve_transfer_backend(True, None) == "kernel"
    assert resolve_transfer_backend(False, None) == "direct"
    assert resolve_transfer_backend(True, " Direct ") == "direct"
    assert resolve_transfer_backend(False, "KERNEL") == "kernel"
    with pytest.raises(ValueError, match="expected one of: direct, kernel"):
        resolve_transfer_backend(False, "rdma")


# ---------------------------------------------------------------------------
# Worker-side save-list assembly (worker.py:826-885, 982-1005)
# ---------------------------------------------------------------------------

class _Intent:
    def __init__(self, block_ids_by_group, block_hashes):
        self.block_ids_by_group = block_ids_by_group
        self.block_hashes = block_hashes


def test_block_shard_stripes_are_disjoint_and_complete():
    from pegaflow_amd.connector import block_shard
    ids = [7, 0, 12, 5, 9, 4, 18]
    hashes = [bytes([i]) for i in range(len(ids))]
    assert block_shard(ids, hashes, 0, 1) == (ids, hashes)
    seen = []
    for rank in range(4):
        got_ids, got_hashes = block_shard(ids, hashes, rank, 4)
        assert all(b % 4 == rank for b in got_ids)
        assert [hashes[ids.index(b)] for b in got_ids] == got_hashes     # hashes travel with ids
        seen += got_ids
    assert sorted(seen) == sorted(ids)
    with pytest.raises(ValueError):
        block_shard([1, 2], [b"a"], 0, 2)


def test_assemble_layer_saves_drops_null_blocks_and_follows_groups():
    from pegaflow_amd.connector import assemble_layer_saves
    h = [b"h0", b"h1", b"h2"]
    intents = [
        _Intent([[4, 0, 6], [9, 8, 0]], h),       # group 0 and group 1 ids of one request
        _Intent([[], []], []),                     # nothing to save: skipped
        _Intent([[2], [3]], [b"x"]),
    ]
    got = assemble_layer_saves(intents, ["attn.0", "attn.1", "gdn.0"],
                               layer_to_group={"attn.0": 0, "attn.1": 0, "gdn.0": 1})
    assert got == [
        ("attn.0", [4, 6, 2], [b"h0", b"h2", b"x"]),
        ("attn.1", [4, 6, 2], [b"h0", b"h2", b"x"]),
        ("gdn.0", [9, 8, 3], [b"h0", b"h1", b"x"]),
    ]
    # page-first: each rank keeps its stripe of the non-null blocks
    got = assemble_layer_saves([_Intent([[4, 0, 6, 7]], [b"a", b"b", b"c", b"d"])], ["l0", "l1"],
                               page_first=True, stripe=(1, 2))
    assert got == [("l0", [7], [b"d"]), ("l1", [7], [b"d"])]
    # cross-layer mode: one pseudo-layer whose block is all layers
    got = assemble_layer_saves([_Intent([[1, 2]], [b"a", b"b"])], ["ignored"], cross_layer_key="ALL_LAYERS")
    assert got == [("ALL_LAYERS", [1, 2], [b"a", b"b"])]
    with pytest.raises(RuntimeError, match="save block/hash count mismatch for l0: blocks=2 hashes=1"):
        assemble_layer_saves([_Intent([[1, 2]], [b"a"])], ["l0"])
    with pytest.raises(RuntimeError, match="save intent is missing cache group 1 for l1"):
        assemble_layer_saves([_Intent([[1]], [b"a"])], ["l1"], layer_to_group={"l1": 1})


def test_registration_tensor_accepts_shared_recurrent_states():
    import torch
    from pegaflow_amd.connector import registration_tensor
    t = torch.zeros(8, 16)
    assert registration_tensor(t) is t
    storage = torch.zeros(8 * 24)
    conv = storage.as_strided((8, 16), (24, 1))
    ssm = storage.as_strided((8, 8), (24, 1), 16)
    assert registration_tensor((conv, ssm)) is conv
    with pytest.raises(RuntimeError, match="share one CUDA allocation"):
        registration_tensor((conv, torch.zeros(8, 8)))
    with pytest.raises(RuntimeError, match="same block count"):
        registration_tensor((conv, storage.as_strided((4, 8), (24, 1), 16)))
    with pytest.raises(RuntimeError, match="one common page stride"):
        registration_tensor((conv, storage.as_strided((8, 8), (12, 1), 16)))
    with pytest.raises(TypeError):
        registration_tensor(())


# ---- hybrid hit, storage groups, namespace ------------------------------------
# python/tests/test_hybrid_reconcile.py:38-140 and test_derive_namespace.py:48-72

from types import SimpleNamespace  # noqa: E402

from pegaflow_amd.connector import (derive_namespace, reconcile_hybrid_hit,  # noqa: E402
                                    storage_group_ids)


@pytest.mark.parametrize("attn,recurrent,want", [
    (3, (((2,),),), (3, 2, {2})),                       # rightmost checkpoint within the prefix
    (2, (((2,),),), (0, None, set())),                  # checkpoint beyond the attention prefix
    (3, (((),),), (0, None, set())),                    # attention alone cannot resume
    (4, (((1, 2), (2, 3)),), (3, 2, {2})),              # shards must agree on the boundary
    (3, (((0, 2),), ((1, 2),)), (3, 2, {2})),           # every recurrent group must hold it
    (3, (((0, 2),), ((1,),)), (0, None, set())),
    (3, (((0, 2),),), (3, 2, {0, 2})),                  # a gap below the rightmost hit is fine
    (0, (((0,),),), (0, None, set())),                  # no attention prefix, no hit
    (4, (((1, 3),),), (4, 3, {1, 3})),                  # earlier boundary kept for re-derivation
    (3, (), (0, None, set())),
])
def test_reconcile_hybrid_hit(attn, recurrent, want):
    hit, checkpoint, usable = reconcile_hybrid_hit(attn, recurrent)
    assert (hit, checkpoint, set(usable)) == want
    assert isinstance(usable, frozenset)


def test_storage_group_ids():
    assert storage_group_ids([False, True]) == (0, 1)            # attention first
    assert storage_group_ids([True, False]) == (1, 0)            # recurrent group can come first
    assert storage_group_ids([False]) == (0,)
    assert storage_group_ids([False, True, True]) == (0, 1, 2)   # dense ids for several recurrent groups
    from pegaflow_amd.worker_connector import CacheGroups
    groups = CacheGroups((("mamba",), ("attn",)), frozenset({0}))
    assert groups.storage_group_ids == (1, 0) and groups.hash_group_index == 1
    assert groups.storage_group_of(0) == 1


def _vllm_config(pp_size=1, mla_layer_split=False, disable_hma=False):
    model = SimpleNamespace(model="/data/models/GLM-5.2-FP8", dtype="bfloat16",
                            get_total_num_kv_heads=lambda: 1, get_head_size=lambda: 576,
                            get_total_num_hidden_layers=lambda: 78)
    return SimpleNamespace(
        model_config=model, cache_config=SimpleNamespace(cache_dtype="fp8"),
        scheduler_config=SimpleNamespace(disable_hybrid_kv_cache_manager=disable_hma),
        parallel_config=SimpleNamespace(pipeline_parallel_size=pp_size),
        additional_config={"mla_layer_split_kv_cache": mla_layer_split})


def test_namespace_separates_incompatible_layouts():
    ns = lambda **kw: derive_namespace(_vllm_config(**kw), tp_size=8)  # noqa: E731
    assert ns(pp_size=1) != ns(pp_size=8)
    assert ns(mla_layer_split=False) != ns(mla_layer_split=True)
    assert ns(disable_hma=False) != ns(disable_hma=True)
    assert ns(pp_size=4, mla_layer_split=True) == ns(pp_size=4, mla_layer_split=True)
    cfg = _vllm_config(pp_size=4)
    cfg.additional_config = None
    assert derive_namespace(cfg, tp_size=8) == ns(pp_size=4, mla_layer_split=False)
    assert derive_namespace(_vllm_config(), tp_size=8) != derive_namespace(_vllm_config(), tp_size=4)
    assert derive_namespace(_vllm_config(), 8, dcp_world_size=2) != ns()
    assert derive_namespace(_vllm_config(), 8, cross_layer_blocks=True) != ns()
    value = ns()
    assert len(value) == 8 and int(value, 16) >= 0
