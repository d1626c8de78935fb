"""Wire format of the gRPC messages on the save / load path: the descriptors
are built in code (there is no protoc in the image), so the encodings are
checked against bytes written out by hand from the field numbers and types of
the reference's pegaflow-proto/proto/engine.proto:22-176 and the protobuf
encoding rules (tag = field << 3 | wire type; packed repeated scalars)."""

import pytest

grpc = pytest.importorskip("grpc")

from pegaflow_amd import rpc  # noqa: E402


def test_save_request_bytes():
    req = rpc.SaveRequest(instance_id="i", tp_rank=2, device_id=1, pp_rank=3,
                          saves=[rpc.SaveLayer(layer_name="L", block_ids=[1, 300],
                                               block_hashes=[b"\x01\x02"])])
    want = bytes.fromhex("0a0169" "1002" "1801"
                         "220c" "0a014c" "120301ac02" "1a020102"
                         "2803")
    assert req.SerializeToString() == want
    back = rpc.SaveRequest.FromString(want)
    assert list(back.saves[0].block_ids) == [1, 300] and back.pp_rank == 3


def test_register_context_request_field_numbers():
    req = rpc.RegisterContextRequest(
        instance_id="a", namespace="n", tp_rank=1, tp_size=2, world_size=4, device_id=3,
        layer_names=["l"], wrapper_bytes=[b"\xff"], num_blocks=[5], bytes_per_block=[6],
        kv_stride_bytes=[7], segments=[2], pp_rank=1, client_version="v", transfer_mode=1,
        page_first=True, layer_group_ids=[0, 1])
    want = bytes.fromhex("0a0161" "12016e" "1801" "2002" "2804" "3003"
                         "42016c" "4a01ff" "520105" "5a0106" "620107" "6a0102"
                         "7001" "7a0176" "880101" "900101" "9a01020001")
    assert req.SerializeToString() == want


def test_load_request_absent_target_and_lease():
    req = rpc.LoadRequest(instance_id="a", tp_rank=1, load_state_shm="x",
                          groups=[rpc.LoadGroup(layer_names=["l0", "l1"])])
    ll = req.loads.add(lease=rpc.lease_to_bytes(7))
    group = ll.block_ids_by_group.add()
    group.targets.add().block_id = 0     # a present target whose id is 0 is still on the wire
    group.targets.add()                  # absent target
    group.targets.add().block_id = 5
    want = bytes.fromhex("0a0161" "1001" "220178" "2a08" "0a026c30" "0a026c31"
                         "321e" "0a10" "0700000000000000" "0000000000000000"
                         "120a" "0a020800" "0a00" "0a020805")
    assert req.SerializeToString() == want
    back = rpc.LoadRequest.FromString(want)
    targets = back.loads[0].block_ids_by_group[0].targets
    assert [t.block_id if t.HasField("block_id") else None for t in targets] == [0, None, 5]
    assert rpc.lease_from_bytes(back.loads[0].lease) == 7


def test_query_response_oneof():
    ready = rpc.QueryResponse(ready=rpc.QueryReadyMsg(num_hit_blocks=3, lease=b"x" * 16,
                                                   hit_positions=[0, 2]))
    assert ready.SerializeToString() == bytes.fromhex("1218" "0803" "1210" + "78" * 16 + "1a020002")
    loading = rpc.QueryResponse(loading=rpc.QueryLoadingMsg())
    assert loading.SerializeToString() == bytes.fromhex("0a00")
    assert rpc.QueryResponse.FromString(bytes.fromhex("0a00")).WhichOneof("outcome") == "loading"


def test_lease_bytes_rules():
    """lease.rs:22-31."""
    with pytest.raises(ValueError, match="query lease id must be non-empty"):
        rpc.lease_from_bytes(b"")
    with pytest.raises(ValueError, match="query lease id must be 16 bytes, got 3"):
        rpc.lease_from_bytes(b"abc")
    assert rpc.lease_from_bytes(rpc.lease_to_bytes(2 ** 40 + 9)) == 2 ** 40 + 9
