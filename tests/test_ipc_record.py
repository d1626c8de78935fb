"""The wire form of HipIPCWrapper (the record a worker sends in
`wrapper_bytes`, in place of the reference's pickled CudaIPCWrapper,
python/pegaflow/ipc_wrapper.py:102-160): a fixed part the C side reads and a
JSON tail with the tensor's shape, stride and storage offset.  Nothing in it is
executed on the receiving side; malformed records are refused.  No GPU needed:
the records are built by hand."""

import pytest

from pegaflow_amd import _lib
from pegaflow_amd.ipc import _FIXED, _MAGIC, HipIPCWrapper, context_key


def _record(shape=(2, 8, 16), stride=(256, 16, 1), offset=4096, size=1 << 20):
    w = HipIPCWrapper.__new__(HipIPCWrapper)
    w.handle = bytes(range(64))
    w.alloc_size = 1 << 21
    w.offset = offset
    w.size_bytes = size
    w.device_uuid = bytes(range(100, 116))
    w.dtype = "bfloat16"
    w.shape = tuple(shape)
    w.stride = tuple(stride)
    w.storage_offset = 0
    return w


def test_round_trip_keeps_every_field():
    w = _record()
    raw = w.to_bytes()
    back = HipIPCWrapper.from_bytes(raw)
    assert back == w
    assert (back.shape, back.stride, back.dtype) == ((2, 8, 16), (256, 16, 1), "bfloat16")
    # padded storage: the stride says more than the shape (ipc_wrapper.py:150-158)
    padded = _record(shape=(4, 100), stride=(128, 1))
    assert HipIPCWrapper.from_bytes(padded.to_bytes()).stride == (128, 1)
    assert HipIPCWrapper.from_bytes(padded.to_bytes()) != w


def test_c_record_is_the_fixed_part():
    w = _record()
    rec = w.c_record()
    assert bytes(rec.handle) == w.handle and bytes(rec.device_uuid) == w.device_uuid
    assert (rec.alloc_size, rec.offset, rec.size_bytes) == (1 << 21, 4096, 1 << 20)
    assert isinstance(rec, _lib.PfIpcTensor)


def test_malformed_records_are_refused():
    raw = _record().to_bytes()
    with pytest.raises(ValueError, match="too short"):
        HipIPCWrapper.from_bytes(raw[:40])
    with pytest.raises(ValueError, match="not a HipIPCWrapper record"):
        HipIPCWrapper.from_bytes(b"\x80\x04" + raw[2:])      # e.g. a pickle
    with pytest.raises(ValueError, match="truncated"):
        HipIPCWrapper.from_bytes(raw[:-3])
    with pytest.raises(ValueError, match="truncated"):
        HipIPCWrapper.from_bytes(raw + b"x")
    # a tail that is not the expected JSON object fails in the parser, not later
    w = _record()
    bad_tail = b"[1, 2, 3]"
    forged = _FIXED.pack(_MAGIC, w.handle, w.alloc_size, w.offset, w.size_bytes, w.device_uuid,
                         len(bad_tail)) + bad_tail
    with pytest.raises(ValueError, match="malformed metadata"):
        HipIPCWrapper.from_bytes(forged)


def test_context_key_form():
    # pegaflow-server/src/service.rs:74-76
    assert context_key("inst", 1, 0, 3) == "inst:tp1:pp0:dev3"
