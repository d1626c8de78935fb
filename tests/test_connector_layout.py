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
