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
