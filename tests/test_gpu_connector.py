"""The worker-side callers on real tensors: a vLLM-shaped KV cache is
registered through ``register_kv_caches`` (shape inference -> engine
registration), save intents become per-layer lists through
``assemble_layer_saves`` (null block dropped), and the blocks come back by
query + load into a second instance.  Checked with torch indexing."""

import pytest

from pegaflow_amd.connector import assemble_layer_saves, register_kv_caches
from pegaflow_amd.engine import LayerSave, PegaEngine

pytestmark = pytest.mark.gpu


class Intent:
    def __init__(self, block_ids_by_group, block_hashes):
        self.block_ids_by_group = block_ids_by_group
        self.block_hashes = block_hashes


@pytest.mark.parametrize("kind", ["kv_first", "mla_page_first"])
def test_register_save_query_load_on_torch_tensors(kind, gpu):
    import torch
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    names = [f"model.layers.{i}.self_attn.attn" for i in range(3)]
    if kind == "kv_first":
        shape, is_mla, page_first = (2, 64, 16, 8, 128), False, False      # [2, blocks, 16, 8, 128]
    else:
        shape, is_mla, page_first = (64, 64, 576), True, True              # MLA latent [blocks, 64, 576]
    src = {n: torch.randn(shape, device=dev, dtype=torch.bfloat16, generator=gen) for n in names}
    dst = {n: torch.zeros(shape, device=dev, dtype=torch.bfloat16) for n in names}
    torch.cuda.synchronize()
    eng = PegaEngine(pool_size=64 << 20)
    try:
        for inst, caches in (("src", src), ("dst", dst)):
            got = register_kv_caches(eng, inst, "ns", 0, caches, 64 if is_mla else 16, is_mla=is_mla,
                                     page_first=page_first)
            assert got == names
        hashes = [bytes([i]) * 8 for i in range(6)]
        intents = [Intent([[5, 0, 9]], hashes[:3]), Intent([[33, 2, 0]], hashes[3:])]
        saves = assemble_layer_saves(intents, names, page_first=page_first,
                                     stripe=(0, 1) if page_first else None)
        assert [s[1] for s in saves] == [[5, 9, 33, 2]] * 3          # null block dropped
        kept_hashes = saves[0][2]
        eng.batch_save_kv_blocks("src", 0, 0, 0, [LayerSave(*s) for s in saves])
        hits, lease = eng.query_prefix("dst", kept_hashes)
        assert hits == 4
        dest = [10, 11, 12, 13]
        eng.batch_load_kv_blocks_multi_layer("dst", 0, 0, [names], lease, [dest]).wait()
        block_dim = 1 if kind == "kv_first" else 0
        for n in names:
            want = torch.zeros_like(src[n])
            want.index_copy_(block_dim, torch.tensor(dest, device=dev),
                             src[n].index_select(block_dim, torch.tensor([5, 9, 33, 2], device=dev)))
            assert torch.equal(dst[n].view(torch.int16), want.view(torch.int16)), n
    finally:
        eng.close()


@pytest.mark.parametrize("kind", ["kv_first", "mla_page_first", "cross_layer"])
def test_worker_connector_steps_over_a_real_engine(kind, gpu):
    """Two workers (a prefill and a decode instance of one namespace) driven the
    way vLLM drives them: metadata in, start_load_kv / wait_for_save per step,
    get_finished polled until the requests are reported."""
    import time

    import torch

    from pegaflow_amd.worker_connector import (ConnectorContext, InProcessEngineClient, LoadIntent,
                                               PegaConnectorMetadata, SaveIntent, WorkerConnector)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)
    names = [f"model.layers.{i}.self_attn.attn" for i in range(4)]
    if kind == "kv_first":
        shape, is_mla, block_size, block_dim = (2, 96, 16, 8, 128), False, 16, 1
    elif kind == "mla_page_first":
        shape, is_mla, block_size, block_dim = (96, 64, 576), True, 64, 0
    else:
        # one tensor for all layers: [blocks, layers, K/V, tokens, heads, head size]
        shape, is_mla, block_size, block_dim = (96, 3, 2, 16, 4, 64), False, 16, 0
        names = ["ALL_LAYERS"]
    src = {n: torch.randn(shape, device=dev, dtype=torch.bfloat16, generator=gen) for n in names}
    dst = {n: torch.zeros(shape, device=dev, dtype=torch.bfloat16) for n in names}
    torch.cuda.synchronize()
    eng = PegaEngine(pool_size=64 << 20)
    client = InProcessEngineClient(eng)

    def worker_for(instance):
        ctx = ConnectorContext(instance_id=instance, namespace="ns", block_size=block_size,
                               tp_size=1, world_size=1, tp_rank=0, device_id=0,
                               engine_client=client, is_mla=is_mla)
        return WorkerConnector(ctx, device_synchronize=torch.cuda.synchronize)

    def poll(worker, finished, which, want, seconds=20.0):
        deadline = time.time() + seconds
        seen = set()
        while time.time() < deadline:
            got = worker.get_finished(finished)[which]
            finished = set()
            seen |= got or set()
            if seen == want:
                return
            time.sleep(0.002)
        raise AssertionError(f"{want - seen} never reported")

    prefill, decode = worker_for("prefill"), worker_for("decode")
    try:
        if kind == "cross_layer":
            prefill.register_cross_layers_kv_cache(src["ALL_LAYERS"])
            decode.register_cross_layers_kv_cache(dst["ALL_LAYERS"])
        else:
            prefill.register_kv_caches(src)
            decode.register_kv_caches(dst)
        assert prefill._registered_layers == names and prefill._page_first == is_mla
        # step 1: two requests finish prefill; request b holds the null block
        hashes_a = [b"a%d" % i + bytes(6) for i in range(5)]
        hashes_b = [b"b%d" % i + bytes(6) for i in range(3)]
        step = PegaConnectorMetadata(save_intents={
            "a": SaveIntent(((7, 3, 50, 51, 9),), tuple(hashes_a)),
            "b": SaveIntent(((0, 20, 21),), tuple(hashes_b))})
        prefill.start_load_kv(step)
        prefill.save_kv_layer(step, names[0], src[names[0]], None)     # per-layer hook: nothing
        prefill.wait_for_save()
        poll(prefill, {"a", "b"}, 0, {"a", "b"})
        assert eng.cached_blocks == 7                                # b's null block was dropped
        # step 2: the scheduler side queries, the decode worker loads
        hits, lease = client.query("decode", hashes_a)
        assert hits == 5
        hits_b, lease_b = client.query("decode", hashes_b)
        assert hits_b == 0 and lease_b == b""                          # b's first block was never stored
        dest = (60, 61, None, 63, 64)
        decode.start_load_kv(PegaConnectorMetadata(load_intents={
            "a": LoadIntent((dest,), (lease,), num_tokens=5 * block_size)}))
        decode.wait_for_layer_load(names[0])
        poll(decode, set(), 1, {"a"})
        assert decode.get_block_ids_with_load_errors() == set()
        src_ids = torch.tensor([7, 3, 51, 9], device=dev)
        dst_ids = torch.tensor([60, 61, 63, 64], device=dev)
        for n in names:
            want = torch.zeros_like(src[n])
            want.index_copy_(block_dim, dst_ids, src[n].index_select(block_dim, src_ids))
            assert torch.equal(dst[n].view(torch.int16), want.view(torch.int16)), n
        # step 3: a lease the engine does not know fails the load call; vLLM is told to recompute
        decode.start_load_kv(PegaConnectorMetadata(load_intents={
            "c": LoadIntent(((70, 71),), (client.lease_token(987654),), num_tokens=2 * block_size)}))
        assert decode.get_block_ids_with_load_errors() == {70, 71}
        assert decode.get_finished(set())[1] == {"c"}
    finally:
        prefill.shutdown()
        decode.shutdown()
        eng.close()


def test_hybrid_worker_resumes_attention_prefix_and_recurrent_checkpoint(gpu):
    """A hybrid model (attention + recurrent state) through two workers: the
    attention group saves a three-block prefix, the recurrent group only the
    checkpoint at its end; the scheduler-side facts (prefix hit, per-group
    membership, reconcile_hybrid_hit) turn into one load with a prefix lease and
    a membership lease (worker.py:572-619, hybrid_groups.rs:14-176)."""
    import time

    import torch

    from pegaflow_amd.connector import reconcile_hybrid_hit
    from pegaflow_amd.worker_connector import (CacheGroups, ConnectorContext,
                                               InProcessEngineClient, LoadIntent,
                                               PegaConnectorMetadata, RecurrentLoadHold,
                                               SaveIntent, WorkerConnector)
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(3)
    blocks, page_elems = 32, 2048                          # one 4 KiB state page per block

    def make_caches(fill):
        caches = {}
        for name in ("attn_0", "attn_1"):
            caches[name] = (torch.randn((2, blocks, 16, 4, 64), device=dev, dtype=torch.bfloat16,
                                        generator=gen) if fill
                            else torch.zeros((2, blocks, 16, 4, 64), device=dev, dtype=torch.bfloat16))
        page = (torch.randn(blocks * page_elems, device=dev, dtype=torch.float16, generator=gen)
                if fill else torch.zeros(blocks * page_elems, device=dev, dtype=torch.float16))
        # two state tensors viewing one page-strided allocation (conv state, ssm state)
        caches["recurrent_state"] = (page.as_strided((blocks, 512), (page_elems, 1), 0),
                                     page.as_strided((blocks, 1024), (page_elems, 1), 512))
        return caches, page

    src, src_page = make_caches(True)
    dst, dst_page = make_caches(False)
    torch.cuda.synchronize()
    groups = CacheGroups((("attn_0", "attn_1"), ("recurrent_state",)), frozenset({1}))
    eng = PegaEngine(pool_size=64 << 20)
    client = InProcessEngineClient(eng)

    def worker_for(instance):
        ctx = ConnectorContext(instance_id=instance, namespace="hybrid", block_size=16, tp_size=1,
                               world_size=1, tp_rank=0, device_id=0, engine_client=client)
        return WorkerConnector(ctx, groups, device_synchronize=torch.cuda.synchronize)

    prefill, decode = worker_for("prefill"), worker_for("decode")
    try:
        prefill.register_kv_caches(src)
        decode.register_kv_caches(dst)
        hashes = [bytes([40 + i]) * 8 for i in range(3)]
        step = PegaConnectorMetadata(save_intents={"r": SaveIntent(
            block_ids_by_group=((1, 2, 3), (0, 0, 9)), block_hashes=tuple(hashes))})
        prefill.start_load_kv(step)
        prefill.wait_for_save()                              # recurrent state: saved before returning
        assert prefill.get_finished({"r"})[0] == {"r"}
        # the scheduler's view
        hits, lease = client.query("decode", hashes)
        members = eng.query_group_membership("decode", groups.storage_group_of(1), hashes)
        assert hits == 3 and members == [False, False, True]
        positions = tuple(i for i, present in enumerate(members) if present)
        hit_blocks, checkpoint, usable = reconcile_hybrid_hit(hits, ((positions,),))
        assert (hit_blocks, checkpoint, usable) == (3, 2, frozenset({2}))
        member_lease = client.lease_token(eng.create_group_lease(
            "decode", groups.storage_group_of(1), [hashes[p] for p in positions]))
        hold = RecurrentLoadHold(leases=((member_lease,),), hit_positions=((positions,),),
                                 checkpoint=checkpoint)
        decode.start_load_kv(PegaConnectorMetadata(load_intents={"r": LoadIntent(
            block_ids_by_group=((11, 12, 13), (None, None, 21)), leases=(lease,), num_tokens=48,
            recurrent_hold=hold)}))
        deadline = time.time() + 20
        done = None
        while done is None and time.time() < deadline:
            done = decode.get_finished(set())[1]
            time.sleep(0.002)
        assert done == {"r"} and decode.get_block_ids_with_load_errors() == set()
        for name in ("attn_0", "attn_1"):
            want = torch.zeros_like(src[name])
            want[:, 11:14] = src[name][:, 1:4]
            assert torch.equal(dst[name].view(torch.int16), want.view(torch.int16)), name
        want_page = torch.zeros_like(src_page).view(blocks, page_elems)
        want_page[21] = src_page.view(blocks, page_elems)[9]
        assert torch.equal(dst_page.view(blocks, page_elems).view(torch.int16),
                           want_page.view(torch.int16))
    finally:
        prefill.shutdown()
        decode.shutdown()
        eng.close()
