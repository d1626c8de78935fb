"""Shared-memory load completion flag (sync_state.rs:23-300 of the reference):
wire format and state transitions, no GPU needed."""

import os
import struct

import pytest

from pegaflow_amd import _lib
from pegaflow_amd.engine import (LOAD_STATE_ERROR, LOAD_STATE_PENDING, LOAD_STATE_SUCCESS,
                                 LoadState)


def test_create_attach_and_signal():
    a = LoadState()
    assert a.shm_name.startswith("pega_load_") and len(a.shm_name) == len("pega_load_") + 32
    assert a.get() == LOAD_STATE_PENDING
    b = LoadState(attach_to=a.shm_name)
    assert b.get() == LOAD_STATE_PENDING
    b.set_completed()
    assert a.get() == LOAD_STATE_SUCCESS
    b.set_error()
    assert a.get() == LOAD_STATE_ERROR
    b.close()
    a.close()


def test_wire_format():
    """First 8 bytes: offset of the record; record = u32 magic 'PFLD', u32
    version 1, i64 state; 32 bytes in all."""
    s = LoadState()
    path = "/dev/shm/" + s.shm_name
    raw = open(path, "rb").read()
    assert len(raw) == 32
    (offset,) = struct.unpack_from("<Q", raw, 0)
    assert offset == 8
    magic, version, state = struct.unpack_from("<IIq", raw, offset)
    assert (magic, version, state) == (0x50464C44, 1, 0)
    s.set_completed()
    raw = open(path, "rb").read()
    assert struct.unpack_from("<q", raw, offset + 8)[0] == 1
    s.close()
    assert not os.path.exists(path)  # the creator unlinks


def test_attach_rejects_foreign_objects(tmp_path):
    with pytest.raises(_lib.StorageError, match="failed to open shared memory"):
        LoadState(attach_to="pega_load_does_not_exist")
    name = "pega_load_test_bad_header_%d" % os.getpid()
    with open("/dev/shm/" + name, "wb") as f:
        f.write(struct.pack("<QIIq", 8, 0x12345678, 1, 0) + b"\0" * 8)
    try:
        with pytest.raises(_lib.StorageError, match="invalid LoadState header"):
            LoadState(attach_to=name)
        with open("/dev/shm/" + name, "wb") as f:
            f.write(b"\0" * 8)
        with pytest.raises(_lib.StorageError, match="too small"):
            LoadState(attach_to=name)
    finally:
        os.unlink("/dev/shm/" + name)
