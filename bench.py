#!/usr/bin/env python3
"""Benchmark of the layer-wise KV block transfer path on one MI355X.

Default workload (BASELINE.json configs[1] + configs[2], Llama-3.1-8B shape):
  32 layers, each a K/V-split paged cache [2, 8192 blocks, 16, 8, 128] bf16
  (N(0,1), seeded); 5,000 blocks (8 requests x 625, a seeded permutation of
  the pool) are SAVED layer by layer into the pinned host pool (gather,
  GPU -> host) and then LOADED into freshly permuted destination block ids of
  a second, zeroed cache (scatter, host -> GPU).

One step = one save pass + one load pass.  `value` = payload bytes of K steps /
wall time of K steps, device inputs and the host pool resident before the
timed region.  Save and load rates, the measured contiguous-copy link peak,
the gather kernel's HBM roofline, the GEMM-overlap run and the CPU baseline
(oracle memcpy executor on host cores) are reported in the same JSON line.

`--workload llama70b_fp8` and `--workload dsv3_mla` run BASELINE configs[3]
and configs[4] through the same harness (extra measurements; the driver's
line is the default workload).
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PCIE_GEN5_X16_GBPS = 63.0   # 32 GT/s x 16 lanes x 128/130 / 8
HBM_PEAK_GBPS = 8000.0      # MI355X published HBM3E bandwidth
# rocprofv3 summaries of the staged gather/scatter kernel, one per workload.  Each
# carries one line `traffic-record: key=value ...` with the HBM bytes a launch
# moved (FETCH_SIZE / WRITE_SIZE per dispatch, scaled by what the same counters
# read for a plain copy of exactly 1 GiB) and the algorithmic bytes of the
# launches it was measured on; `roofline.traffic` is read from there and only
# reported when this run's launches have that same algorithmic size.
TRAFFIC_PROFILES = {
    "llama8b": "block_tiles_rows_kernel_llama8b_save_load.md",
    "llama70b_fp8": "block_tiles_rows_kernel_llama70b_fp8_save_load.md",
    "dsv3_mla": "block_tiles_kernel_dsv3_mla_page_first_save_load.md",
}


def measured_traffic(workload, alg_bytes_per_launch):
    """(bytes per launch, source file) from the committed profile summary of this
    workload, or (None, reason) when there is none for launches of this size."""
    name = TRAFFIC_PROFILES.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None, "no profile summary for this workload"
    rec = None
    with open(path) as f:
        for line in f:
            if line.startswith("traffic-record:"):
                rec = dict(kv.split("=", 1) for kv in line.split()[1:])
    if rec is None:
        return None, f"profiles/{name} has no traffic-record line"
    if abs(float(rec["alg_bytes"]) - alg_bytes_per_launch) > 0.005 * alg_bytes_per_launch:
        return None, (f"profiles/{name} was measured on launches of {rec['alg_bytes']} algorithmic "
                      f"bytes, this run's move {int(alg_bytes_per_launch)}")
    total = (float(rec["fetch_kib"]) * float(rec["fetch_scale"]) +
             float(rec["write_kib"]) * float(rec["write_scale"])) * 1024
    return int(round(total)), f"profiles/{name}"


WORKLOADS = {
    # BASELINE configs[1] (save) + configs[2] (load)
    "llama8b": dict(label="configs[1]+configs[2]: Llama-3.1-8B KV [2,8192,16,8,128] bf16",
                    layers=32, num_blocks=8192, seg=16 * 8 * 128 * 2, split=True, n=5000,
                    dtype="bf16", ids="permutation", page_first=False),
    # BASELINE configs[3]
    "llama70b_fp8": dict(label="configs[3]: Llama-3-70B KV [2,16384,16,8,128] fp8 e4m3",
                         layers=80, num_blocks=16384, seg=16 * 8 * 128, split=True, n=8192,
                         dtype="fp8", ids="runs", page_first=False),
    # BASELINE configs[4]
    "dsv3_mla": dict(label="configs[4]: DeepSeek-V3 MLA latent [4096,64,576] bf16, page-first",
                     layers=61, num_blocks=4096, seg=64 * 576 * 2, split=False, n=2048,
                     dtype="bf16", ids="permutation", page_first=True),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload",
                    choices=sorted(WORKLOADS) + ["ref_transfer_bench", "ref_cpu_path",
                                                 "link_after_free", "launch_fit",
                                                 "fragment_sweep", "unlike_layers"],
                    default="llama8b",
                    help="ref_transfer_bench = the shapes of the reference's own "
                         "benches/transfer_h2d.rs through the descriptor backends; "
                         "ref_cpu_path = the engine-level groups of its benches/cpu_path.rs "
                         "(long lists of 1 KiB blocks through save / query / load); "
                         "link_after_free = what a large hipFree does to the link copies that "
                         "follow it; launch_fit = duration of one staged gather / scatter launch "
                         "against its bytes: the fixed cost of a launch and the steady rate; "
                         "fragment_sweep = rate of the staged gather / scatter launches against "
                         "the fragment size, 1 KiB to 256 KiB; unlike_layers = the staged launches "
                         "of a task whose layers differ in length (cache groups of a hybrid "
                         "model) or in fragment size")
    ap.add_argument("--path", choices=["auto", "staged", "zerocopy"], default="auto")
    ap.add_argument("--layers", type=int, default=0, help="override the layer count")
    ap.add_argument("--slot-mb", type=int, default=0)
    ap.add_argument("--slots", type=int, default=0)
    ap.add_argument("--group-mb", type=int, default=0,
                    help="staged layers that follow one another share a slot and a launch up to "
                         "this size (pf_xfer_config.staged_group_bytes; default: the slot size)")
    ap.add_argument("--unroll", type=int, default=0)
    ap.add_argument("--zc-max-wg", type=int, default=0)
    ap.add_argument("--copy-stream", type=int, default=0, choices=[0, 1, 2],
                    help="staged path: 0 default, 1 link copies on a side stream, 2 in order on "
                         "the caller's stream (kernels then never overlap a copy)")
    ap.add_argument("--no-overlap", action="store_true", help="skip the GEMM-overlap section")
    ap.add_argument("--engine-side-streams", action="store_true",
                    help="engine section: workers move their link copies on a second stream each "
                         "(pf_engine_config.side_copy_streams)")
    ap.add_argument("--gemm-m", type=int, default=4096,
                    help="edge of the square bf16 GEMMs of the overlap section (BASELINE: 4096)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-engine", action="store_true", help="skip the save/query/load engine section")
    ap.add_argument("--engine-mode", choices=["direct", "kernel", "zerocopy"], default="direct",
                    help="transfer mode the engine section registers its instances with "
                         "(zerocopy = PF_MODE_ZEROCOPY: the block-ID engine pinned to the "
                         "zero-copy kernel)")
    ap.add_argument("--engine-descriptors", action="store_true",
                    help="engine section: the workers build one descriptor per fragment and call "
                         "the descriptor backends, as the reference's workers do")
    ap.add_argument("--engine-child", action="store_true",
                    help="(internal) run only the engine section and print its JSON")
    ap.add_argument("--engine-lazy-staging", action="store_true",
                    help="engine section: the workers allocate their staging slots on the first "
                         "staged task instead of at registration (pf_engine_config.lazy_staging)")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--ref-fragments", type=int, default=0,
                    help="ref_transfer_bench: only this fragment count (default: 1024..65536)")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--settle-max", type=int, default=8,
                    help="upper bound on the untimed passes run after the warmup until two agree")
    ap.add_argument("--no-extra-workloads", action="store_true",
                    help="default run only: skip the configs[3] and configs[4] workloads that "
                         "follow the headline one (the `workloads` key)")
    ap.add_argument("--free-gib", type=int, nargs="+", default=[10, 20, 40],
                    help="link_after_free: GiB of device memory to allocate, touch and free")
    return ap.parse_args()


def make_ids(np, kind, num_blocks, n, seed):
    """Block ids of a workload: a seeded permutation prefix, or (configs[3])
    half in contiguous runs of length 8..64 and half isolated, runs and
    singles interleaved in random order."""
    rng = np.random.default_rng(seed)
    if kind == "permutation":
        return rng.permutation(num_blocks)[:n].astype(np.uint32)
    taken = np.zeros(num_blocks, dtype=bool)
    pieces = []
    in_runs = 0
    while in_runs < n // 2:
        length = int(min(rng.integers(8, 65), n // 2 - in_runs))
        start = int(rng.integers(0, num_blocks - length))
        if taken[start:start + length].any():
            continue
        taken[start:start + length] = True
        pieces.append(np.arange(start, start + length))
        in_runs += length
    free = np.flatnonzero(~taken)
    singles = rng.choice(free, n - in_runs, replace=False)
    pieces += [np.array([s]) for s in singles]
    order = rng.permutation(len(pieces))
    return np.concatenate([pieces[i] for i in order]).astype(np.uint32)


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (the path has no inter-GPU step); "
              f"--gpus {args.gpus} is not supported", file=sys.stderr)
        sys.exit(2)
    if args.workload == "ref_cpu_path":  # a native program; nothing here touches the GPU
        run_ref_cpu_path()
        return

    import numpy as np
    import torch

    from pegaflow_amd import runtime

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    runtime.set_device(0)

    if args.workload == "ref_transfer_bench":
        run_ref_transfer_bench(torch, np, args)
        return
    if args.workload == "link_after_free":
        print(json.dumps(run_link_after_free(runtime, args.free_gib)))
        return
    if args.workload == "launch_fit":
        print(json.dumps(run_launch_fit(torch, np, runtime)))
        return
    if args.workload == "fragment_sweep":
        print(json.dumps(run_fragment_sweep(torch, np, runtime)))
        return
    if args.workload == "unlike_layers":
        print(json.dumps(run_unlike_layers(torch, np, runtime)))
        return
    if args.engine_child:
        print(json.dumps(run_workload(args, args.workload, {"engine_child"}, torch, np)))
        return
    sections = set()
    if not args.no_overlap:
        sections |= {"overlap", "duplex"}
    if not args.no_engine:
        sections.add("engine")
    if not args.no_cpu:
        sections.add("cpu")
    result = run_workload(args, args.workload, sections, torch, np)
    # The other two GPU configurations of the benchmark in the same run, as the
    # reference's own transfer bench sweeps its shapes in one run
    # (benches/transfer_h2d.rs:62-109): timed steps, byte check, link and kernel
    # roofline each; the headline keys above stay those of the first workload.
    default_run = (args.workload == "llama8b" and args.path == "auto" and not args.layers
                   and not args.no_extra_workloads)
    if default_run:
        keys = ("value", "save_gbps", "load_gbps", "ms_per_step", "step_save_load_ms",
                "settle_steps", "config", "roofline", "link", "byte_checks", "verified")
        workloads = {"llama8b": {k: result[k] for k in keys}}
        freed = result["device_bytes_released"]
        for name in ("llama70b_fp8", "dsv3_mla"):
            pause = pause_after_free(runtime, freed)
            extra = run_workload(args, name, set(), torch, np)
            workloads[name] = {k: extra[k] for k in keys}
            workloads[name]["pause_after_previous_workload"] = pause
            freed = extra["device_bytes_released"]
        result["workloads"] = workloads
    print(json.dumps(result))


_LINK_CHECK = {}
# The driver clears freed device memory at 28.5 GiB/s on MI355X (`--workload
# link_after_free`: 10 / 20 / 40 / 80 GiB freed -> copies of the affected stream
# slow for 0.34 / 0.70 / 1.40 / 2.82 s); the pause allows 45 ms per GiB.
CLEARING_S_PER_GIB = 0.045


def link_check(runtime):
    """Rates of one 256 MiB copy each way on a fresh pair of streams set up the
    way a worker pool sets up its pair (the first host -> device copy of one
    stream issued while device -> host copies of the other are in flight): that
    second stream is the one whose copies share a DMA engine with the driver's
    clearing of freed device memory."""
    from pegaflow_amd.runtime import DeviceBuffer, Event, PinnedMemory, Stream
    size = 256 << 20
    if not _LINK_CHECK:   # kept for the life of the process: freeing them is a free, too
        _LINK_CHECK.update(pin=PinnedMemory(2 * size), dev=DeviceBuffer(2 * size),
                           ev=[Event(timing=True) for _ in range(4)])
    pin, dev, ev = _LINK_CHECK["pin"], _LINK_CHECK["dev"], _LINK_CHECK["ev"]
    sa, sb = Stream(), Stream()
    for _ in range(6):
        runtime.memcpy_d2h_async(pin.host_ptr, dev.ptr, 32 << 20, sa)
    for _ in range(3):
        runtime.memcpy_h2d_async(dev.ptr + size, pin.host_ptr + size, 32 << 20, sb)
    sa.synchronize()
    sb.synchronize()
    ev[0].record(sa)
    runtime.memcpy_d2h_async(pin.host_ptr, dev.ptr, size, sa)
    ev[1].record(sa)
    ev[1].synchronize()
    ev[2].record(sb)
    runtime.memcpy_h2d_async(dev.ptr + size, pin.host_ptr + size, size, sb)
    ev[3].record(sb)
    ev[3].synchronize()
    out = {"d2h_gbps": round(size / ev[0].elapsed_ms(ev[1]) / 1e6, 2),
           "h2d_gbps": round(size / ev[2].elapsed_ms(ev[3]) / 1e6, 2)}
    sa.close()
    sb.close()
    return out


def pause_after_free(runtime, freed_bytes):
    """Let the driver finish clearing the device memory this process just freed
    before anything is timed: until then, copies of streams that share the
    clearing's DMA engine (a worker pool's load stream does) run at half rate,
    which says nothing about the transfer path.  Sleeps for the time the
    clearing takes at its measured rate, then checks the link with a fresh
    stream pair (and sleeps on, bounded, if that still reads slow).  No
    workload bytes move."""
    gib = freed_bytes / 2 ** 30
    t0 = time.perf_counter()
    time.sleep(CLEARING_S_PER_GIB * gib)
    check = link_check(runtime)
    while check["h2d_gbps"] < 0.9 * check["d2h_gbps"] and time.perf_counter() - t0 < 15.0:
        time.sleep(0.1)
        check = link_check(runtime)
    return {"freed_gib": round(gib, 1), "paused_ms": round((time.perf_counter() - t0) * 1e3, 1),
            "link_after_pause": check}


def run_link_after_free(runtime, gib_list):
    """What a large hipFree does to the link copies that follow it.  For each
    size: allocate, touch and free that many GiB of device memory, then create
    six fresh streams and time 64 MiB copies each way on every one of them in
    turn (one copy in flight at a time) for a few seconds.  The driver clears
    freed device memory with a DMA engine; a stream whose copies the runtime
    placed on that engine runs at half rate until the clearing is done, the
    others are not affected.  Reports, per size, which streams and directions
    were slowed and until when: freed bytes / that time is the clearing rate."""
    from pegaflow_amd.runtime import DeviceBuffer, Event, PinnedMemory, Stream
    piece = 64 << 20
    n_streams = 6
    pin, dev = PinnedMemory(2 * piece), DeviceBuffer(2 * piece)
    ev = [Event(timing=True) for _ in range(3)]

    def sample(streams, seconds):
        rows, t0 = [], time.perf_counter()
        while time.perf_counter() - t0 < seconds:
            for i, st in enumerate(streams):
                ev[0].record(st)
                runtime.memcpy_d2h_async(pin.host_ptr, dev.ptr, piece, st)
                ev[1].record(st)
                runtime.memcpy_h2d_async(dev.ptr + piece, pin.host_ptr + piece, piece, st)
                ev[2].record(st)
                ev[2].synchronize()
                rows.append((time.perf_counter() - t0, i, ev[0].elapsed_ms(ev[1]),
                             ev[1].elapsed_ms(ev[2])))
        return rows

    warm = [Stream() for _ in range(2)]
    sample(warm, 0.2)
    base = sample(warm, 0.3)
    norm_d2h = sorted(r[2] for r in base)[len(base) // 2]
    norm_h2d = sorted(r[3] for r in base)[len(base) // 2]
    out_rows = []
    for gib in gib_list:
        bufs = []
        for i in range(gib):
            b = DeviceBuffer(1 << 30)
            b.fill(i + 1)
            bufs.append(b)
        runtime.device_synchronize()
        t0 = time.perf_counter()
        for b in bufs:
            b.close()
        free_s = time.perf_counter() - t0
        streams = [Stream() for _ in range(n_streams)]
        # the first two as a worker pool primes its pair: the first host -> device
        # copy of one stream issued while device -> host copies of the other run
        for _ in range(6):
            runtime.memcpy_d2h_async(pin.host_ptr, dev.ptr, piece // 2, streams[0])
        for _ in range(3):
            runtime.memcpy_h2d_async(dev.ptr + piece, pin.host_ptr + piece, piece // 2, streams[1])
        streams[0].synchronize()
        streams[1].synchronize()
        rows = sample(streams, max(2.0, 0.1 * gib))
        slow_h2d = [r for r in rows if r[3] > 1.3 * norm_h2d]
        slow_d2h = [r for r in rows if r[2] > 1.3 * norm_d2h]
        last = max([r[0] for r in slow_h2d + slow_d2h], default=0.0)
        out_rows.append({
            "freed_gib": gib, "free_call_s": round(free_s, 3),
            "streams_with_slow_h2d": sorted({r[1] for r in slow_h2d}),
            "streams_with_slow_d2h": sorted({r[1] for r in slow_d2h}),
            "slow_copy_ms_median": round(sorted([r[3] for r in slow_h2d] + [r[2] for r in slow_d2h])
                                         [(len(slow_h2d) + len(slow_d2h)) // 2], 2)
            if slow_h2d or slow_d2h else None,
            "last_slow_copy_at_s": round(last, 2),
            "clearing_gib_per_s": round(gib / last, 1) if last > 0 else None})
        for st in streams:
            st.close()
        time.sleep(1.0)
    return {"metric": "link copies after hipFree", "unit": "ms per 64 MiB copy",
            "normal": {"h2d_ms": round(norm_h2d, 3), "d2h_ms": round(norm_d2h, 3)},
            "rows": out_rows, "device": runtime.device_name(0)}


def run_launch_fit(torch, np, runtime):
    """Duration of one staged gather and one staged scatter launch against the
    bytes it moves: Llama-shaped layers ([2, 8192, 32 KiB]), 512 to 8192 shuffled
    blocks per launch, every launch running alone (link copies in order on the
    kernels' stream) and bracketed by HIP events; the rotation over eight caches
    keeps a launch from finding the previous one's lines.  A straight line through
    the points gives the fixed cost of a launch (ramp, tail and the event
    bracket, whose own reading is reported) and the steady rate."""
    from pegaflow_amd.layout import KVCacheLayout
    from pegaflow_amd.runtime import Event, PinnedMemory, Stream
    from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath
    dev = torch.device("cuda:0")
    nb, seg, n_caches = 8192, 32768, 8
    caches = [torch.empty(2 * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256)
              for _ in range(n_caches)]
    pool = PinnedMemory(2 * nb * seg)
    stream = Stream()
    xfer = BlockTransfer(copy_stream=2)
    xfer.set_kernel_timing(1)
    rng = np.random.default_rng(0)
    rows = []
    for n in (512, 1024, 2048, 4096, 6144, 8192):
        ids = rng.permutation(nb)[:n].astype(np.uint32)
        per = {"save": [], "load": []}
        for rep in range(2 + 2 * n_caches):
            cache = caches[rep % n_caches]
            layer = [LayerBlocks(layout=KVCacheLayout(cache.data_ptr(), 2 * nb * seg, nb, seg, nb * seg, 2),
                                 block_ids=ids, host=(pool.host_ptr, pool.host_ptr + n * seg),
                                 host_device=(pool.device_ptr, pool.device_ptr + n * seg),
                                 host_len=(n * seg, n * seg), host_stride=seg)]
            for name, fn in (("save", xfer.save), ("load", xfer.load)):
                fn(layer, stream, TransferPath.STAGED)
                stream.synchronize()
                ms, launches = xfer.last_kernel_ms()
                assert launches == 1
                if rep >= 2:
                    per[name].append(ms * 1e3)
        med = {k: sorted(v)[len(v) // 2] for k, v in per.items()}
        rows.append({"blocks": n, "alg_bytes": 4 * n * seg, "gather_us": round(med["save"], 2),
                     "scatter_us": round(med["load"], 2),
                     "gather_gbps": round(4 * n * seg / med["save"] / 1e3, 1),
                     "scatter_gbps": round(4 * n * seg / med["load"] / 1e3, 1)})
    pair = [Event(timing=True), Event(timing=True)]
    empty = []
    for _ in range(50):
        pair[0].record(stream)
        pair[1].record(stream)
        pair[1].synchronize()
        empty.append(pair[0].elapsed_ms(pair[1]) * 1e3)
    fits = {}
    x = np.array([r["alg_bytes"] for r in rows], dtype=np.float64)
    for key in ("gather_us", "scatter_us"):
        y = np.array([r[key] for r in rows])
        slope, intercept = np.polyfit(x, y, 1)
        fits[key[:-3]] = {"fixed_us": round(float(intercept), 2),
                          "steady_gbps": round(1.0 / slope / 1e3, 1),
                          "max_residual_us": round(float(np.abs(y - (slope * x + intercept)).max()), 2)}
    xfer.close()
    stream.close()
    pool.close()
    return {"metric": "staged launch duration against bytes", "unit": "us",
            "rows": rows, "fit": fits, "empty_event_pair_us": round(sorted(empty)[len(empty) // 2], 2),
            "note": "fixed_us includes the event bracket (empty_event_pair_us)",
            "device": runtime.device_name(0)}


def run_fragment_sweep(torch, np, runtime):
    """HBM rate of the staged gather / scatter launches against the fragment
    size: eight K/V-split layers of 320 MiB payload per call (512 MiB staging
    fills, five launches per direction), shuffled ids, every launch running alone
    and bracketed by HIP events (the launch gap is inside the figure); one layer
    of every size is checked block by block."""
    from pegaflow_amd.layout import KVCacheLayout
    from pegaflow_amd.runtime import PinnedMemory, Stream
    from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath
    dev = torch.device("cuda:0")
    n_layers, target = 8, 320 << 20
    pool = PinnedMemory(n_layers * target)
    stream = Stream()
    xfer = BlockTransfer()
    xfer.set_kernel_timing(1)
    rng = np.random.default_rng(0)
    rows = []
    for seg in (1024, 2048, 4096, 8192, 16384, 32768, 65536, 131072, 262144):
        n = target // (2 * seg)
        nb = int(n * 1.6)
        src = [torch.empty(2 * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256)
               for _ in range(n_layers)]
        dst = [torch.zeros(2 * nb * seg, device=dev, dtype=torch.uint8) for _ in range(n_layers)]
        torch.cuda.synchronize()
        save_ids = rng.permutation(nb)[:n].astype(np.uint32)
        load_ids = rng.permutation(nb)[:n].astype(np.uint32)

        def layers(caches, ids):
            out = []
            for li, t in enumerate(caches):
                off = li * 2 * n * seg
                out.append(LayerBlocks(
                    layout=KVCacheLayout(t.data_ptr(), 2 * nb * seg, nb, seg, nb * seg, 2),
                    block_ids=ids, host=(pool.host_ptr + off, pool.host_ptr + off + n * seg),
                    host_device=(pool.device_ptr + off, pool.device_ptr + off + n * seg),
                    host_len=(n * seg, n * seg), host_stride=seg, layer_name=f"l{li}"))
            return out

        sv, ld = layers(src, save_ids), layers(dst, load_ids)
        for _rep in range(3):
            xfer.save(sv, stream, TransferPath.STAGED)
            stream.synchronize()
            save_ms, save_launches = xfer.last_kernel_ms()
            xfer.load(ld, stream, TransferPath.STAGED)
            stream.synchronize()
            load_ms, load_launches = xfer.last_kernel_ms()
        got = dst[3].cpu().numpy().reshape(2, nb, seg)
        want = src[3].cpu().numpy().reshape(2, nb, seg)
        if not np.array_equal(got[:, load_ids], want[:, save_ids]):
            print(f"bench.py: fragment sweep, {seg}-byte fragments: bytes differ", file=sys.stderr)
            sys.exit(1)
        alg = 2.0 * n_layers * 2 * n * seg
        rows.append({"fragment_bytes": seg, "blocks_per_layer": n,
                     "launches": [save_launches, load_launches],
                     "gather_gbps": round(alg / save_ms / 1e6, 1),
                     "scatter_gbps": round(alg / load_ms / 1e6, 1),
                     "gather_frac_of_hbm_peak": round(alg / save_ms / 1e6 / HBM_PEAK_GBPS, 3),
                     "scatter_frac_of_hbm_peak": round(alg / load_ms / 1e6 / HBM_PEAK_GBPS, 3)})
        del src, dst, sv, ld
        torch.cuda.empty_cache()
    xfer.close()
    stream.close()
    pool.close()
    return {"metric": "staged gather / scatter rate against the fragment size", "unit": "GB/s",
            "rows": rows, "verified": True, "device": runtime.device_name(0)}


def run_unlike_layers(torch, np, runtime):
    """Device time of the staged gather and scatter of one task whose layers
    are unlike: (a) 48 K/V-split layers of 32 KiB fragments, every sixth with
    625 blocks and the others with 8 (full-attention and sliding-window cache
    groups); (b) 24 one-segment layers of 512 blocks, 72 KiB and 8 KiB
    fragments in turn (latent and indexer caches).  Each task is one staging
    fill; its launches run alone between one pair of HIP events.  `ideal_us` =
    the task's algorithmic bytes at 6.2 TB/s, the steady rate of these kernels."""
    from pegaflow_amd.layout import KVCacheLayout
    from pegaflow_amd.runtime import PinnedMemory, Stream
    from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath, plan_staged_fills
    dev = torch.device("cuda:0")
    stream = Stream()
    rng = np.random.default_rng(0)
    tasks = {
        "layers_of_unlike_length": [(n, 32768, 2) for n in ([8] * 5 + [625]) * 8],
        "layers_of_unlike_fragment_size": [(512, 73728, 1), (512, 8192, 1)] * 12,
    }
    out = {}
    for name, shapes in tasks.items():
        nb = 2048
        src = [torch.empty(nseg * nb * seg, device=dev, dtype=torch.uint8).random_(0, 256)
               for _n, seg, nseg in shapes]
        dst = [torch.zeros(nseg * nb * seg, device=dev, dtype=torch.uint8) for _n, seg, nseg in shapes]
        payload = sum(n * seg * nseg for n, seg, nseg in shapes)
        pool = PinnedMemory(payload)
        save_ids = [rng.permutation(nb)[:n].astype(np.uint32) for n, _s, _g in shapes]
        load_ids = [rng.permutation(nb)[:n].astype(np.uint32) for n, _s, _g in shapes]

        def layers(caches, ids):
            res, off = [], 0
            for t, (n, seg, nseg), lids in zip(caches, shapes, ids):
                kv = nb * seg if nseg == 2 else 0
                res.append(LayerBlocks(
                    layout=KVCacheLayout(t.data_ptr(), nseg * nb * seg, nb, seg, kv, nseg), block_ids=lids,
                    host=tuple(pool.host_ptr + off + g * n * seg for g in range(nseg)),
                    host_device=tuple(pool.device_ptr + off + g * n * seg for g in range(nseg)),
                    host_len=tuple(n * seg for _ in range(nseg)), host_stride=seg))
                off += nseg * n * seg
            return res

        xfer = BlockTransfer(copy_stream=2)
        xfer.set_kernel_timing(1)
        sv, ld = layers(src, save_ids), layers(dst, load_ids)
        for _rep in range(4):
            xfer.save(sv, stream, TransferPath.STAGED)
            stream.synchronize()
            save_ms, _ = xfer.last_kernel_ms()
            xfer.load(ld, stream, TransferPath.STAGED)
            stream.synchronize()
            load_ms, _ = xfer.last_kernel_ms()
        for li in (0, 5, len(shapes) - 1):
            n, seg, nseg = shapes[li]
            got = dst[li].cpu().numpy().reshape(nseg, nb, seg)
            want = src[li].cpu().numpy().reshape(nseg, nb, seg)
            if not np.array_equal(got[:, load_ids[li]], want[:, save_ids[li]]):
                print(f"bench.py: unlike_layers, {name}, layer {li}: bytes differ", file=sys.stderr)
                sys.exit(1)
        _units, fills = plan_staged_fills([n for n, _s, _g in shapes], [s_ * g for _n, s_, g in shapes])
        out[name] = {"layers": len(shapes), "payload_bytes": payload, "fills": fills,
                     "gather_us": round(save_ms * 1e3, 1), "scatter_us": round(load_ms * 1e3, 1),
                     "ideal_us": round(2 * payload / 6.2e6, 1)}
        xfer.close()
        pool.close()
        del src, dst, sv, ld
        torch.cuda.empty_cache()
    stream.close()
    return {"metric": "device time of the staged launches of a task of unlike layers", "unit": "us",
            "tasks": out, "verified": True, "device": runtime.device_name(0)}


def run_workload(args, workload, sections, torch, np):
    """One workload of WORKLOADS end to end: inputs, timed steps, byte check,
    link peak, kernel roofline and the sections asked for ("overlap", "duplex",
    "engine", "cpu"); returns the result line as a dict.  {"engine_child"} runs
    only the engine section in this process and returns its dict."""
    from pegaflow_amd import _lib, runtime
    from pegaflow_amd.layout import KVCacheLayout
    from pegaflow_amd.pool import LayerTopology, WorkerLayers
    from pegaflow_amd.runtime import Event, PinnedMemory, Stream
    from pegaflow_amd.transfer import BlockTransfer, LayerBlocks, TransferPath

    dev = torch.device("cuda:0")
    path = {"auto": TransferPath.AUTO, "staged": TransferPath.STAGED,
            "zerocopy": TransferPath.ZEROCOPY}[args.path]
    w = WORKLOADS[workload]
    n_layers = args.layers or w["layers"]
    nb, seg, n = w["num_blocks"], w["seg"], w["n"]
    nseg = 2 if w["split"] else 1
    layer_bytes = nseg * nb * seg
    payload_per_layer = nseg * n * seg
    payload = payload_per_layer * n_layers
    names = [f"model.layers.{li}.self_attn.attn" for li in range(n_layers)]

    # ---- inputs, resident before timing ----------------------------------
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed)

    def new_cache(fill):
        if w["dtype"] == "bf16":
            t = torch.empty(layer_bytes // 2, device=dev, dtype=torch.bfloat16)
            if fill:
                t.normal_(generator=gen)
            else:
                t.zero_()
            return t
        t = torch.zeros(layer_bytes, device=dev, dtype=torch.uint8)
        if fill:  # random fp8 e4m3 bytes without the NaN encodings 0x7F / 0xFF
            t.random_(0, 256, generator=gen)
            t[(t & 0x7F) == 0x7F] -= 1
        return t

    src_cache = [new_cache(True) for _ in range(n_layers)]
    dst_cache = [new_cache(False) for _ in range(n_layers)]
    save_ids = make_ids(np, w["ids"], nb, n, args.seed)
    load_ids = make_ids(np, "permutation", nb, n, args.seed + 1)
    if "engine_child" in sections:
        torch.cuda.synchronize()
        return run_engine(torch, np, runtime, w, names, src_cache, dst_cache, save_ids, load_ids,
                          payload, args.engine_mode, args.engine_descriptors,
                          args.engine_lazy_staging, args.engine_side_streams)
    t0 = time.time()
    pool = PinnedMemory(payload)
    pool_alloc_s = time.time() - t0
    torch.cuda.synchronize()
    # Whatever ran on this GPU before this process may have freed device memory a
    # moment ago: check the link with a fresh stream pair and wait (bounded) while
    # the driver's clearing of that memory still slows it.
    link_at_start = pause_after_free(runtime, 0)

    def layouts_for(caches):
        kv = nb * seg if w["split"] else 0
        return [KVCacheLayout(t.data_ptr(), layer_bytes, nb, seg, kv, nseg) for t in caches]

    if w["page_first"]:
        # One page per saved block, layers at the offsets the sealed topology
        # assigns (ids follow the byte-wise sorted layer names).
        topo = LayerTopology([WorkerLayers(0, 0, dict(zip(names, layouts_for(src_cache))))],
                             tp_size=1, page_first=True)
        page = topo.shard_page_size(0)
        assert page * n == payload
        offsets = [topo.page_placement(topo.layer_id(nm))[0] for nm in names]
        pages = np.arange(n, dtype=np.uint64) * page

        def layers_for(caches, ids, mem=pool):
            return [LayerBlocks(layout=L, block_ids=ids,
                                page_host=(mem.host_ptr + pages).astype(np.uint64),
                                page_host_device=(mem.device_ptr + pages).astype(np.uint64),
                                page_offset=offsets[li], page_len=page, layer_name=names[li])
                    for li, L in enumerate(layouts_for(caches))]
    else:
        page, offsets = 0, None
        buf = n * seg  # one host segment buffer (K or V) of one layer

        def layers_for(caches, ids, mem=pool):
            out = []
            for li, L in enumerate(layouts_for(caches)):
                off = li * payload_per_layer
                out.append(LayerBlocks(
                    layout=L, block_ids=ids,
                    host=tuple(mem.host_ptr + off + s * buf for s in range(nseg)),
                    host_device=tuple(mem.device_ptr + off + s * buf for s in range(nseg)),
                    host_len=tuple(buf for _ in range(nseg)), host_stride=seg,
                    layer_name=names[li]))
            return out

    save_layers = layers_for(src_cache, save_ids)
    load_layers = layers_for(dst_cache, load_ids)
    xfer = BlockTransfer(staging_slot_bytes=args.slot_mb << 20, staging_slots=args.slots,
                         tile_unroll=args.unroll, zerocopy_max_workgroups=args.zc_max_wg,
                         copy_stream=args.copy_stream, staged_group_bytes=args.group_mb << 20)
    stream = Stream()
    ev = [Event(timing=True) for _ in range(4)]

    # Every gather / scatter launch of the timed steps is bracketed by HIP events
    # on the stream it runs on (the streams are left as they are); the figures
    # add up over a step and are read after the step's synchronise.
    xfer.set_kernel_timing(2)
    live = {"ms": 0.0, "launches": 0}

    def one_step():
        """save pass + load pass; returns (save_ms, load_ms) from stream events."""
        ev[0].record(stream)
        xfer.save(save_layers, stream, path)
        ev[1].record(stream)
        xfer.load(load_layers, stream, path)
        ev[2].record(stream)
        ev[2].synchronize()
        k_ms, k_n = xfer.last_kernel_ms()
        live["ms"], live["launches"] = live["ms"] + k_ms, live["launches"] + k_n
        return ev[0].elapsed_ms(ev[1]), ev[1].elapsed_ms(ev[2])

    for _ in range(args.warmup):
        one_step()
    # A process that starts right after another one released tens of GiB of
    # device memory (a test run, an earlier bench) can see the driver's clearing
    # of that memory as a second or two of slower passes: the clearing shares a
    # DMA engine with some streams' copies (`--workload link_after_free`).  How
    # much was freed before this process started is not known here, so untimed
    # passes run until two in a row agree (bounded); the count is reported.
    settle_steps, prev = 0, None
    while settle_steps < args.settle_max:
        cur = sum(one_step())
        settle_steps += 1
        if prev is not None and abs(cur - prev) <= 0.015 * min(cur, prev):
            break
        prev = cur
    torch.cuda.synchronize()
    stream.synchronize()
    save_ms = load_ms = 0.0
    step_times = []
    live["ms"], live["launches"] = 0.0, 0
    t_start = time.perf_counter()
    for _ in range(args.steps):
        s_ms, l_ms = one_step()
        save_ms += s_ms
        load_ms += l_ms
        step_times.append((round(s_ms, 2), round(l_ms, 2)))
    stream.synchronize()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t_start
    xfer.set_kernel_timing(0)
    live_launch_ms = live["ms"] / max(live["launches"], 1)
    live_launches_per_step = live["launches"] // max(args.steps, 1)
    used_path = "staged" if xfer.last_path == TransferPath.STAGED else "zerocopy"

    step_bytes = 2 * payload
    value = step_bytes * args.steps / wall / 1e9
    save_gbps = payload * args.steps / (save_ms / 1e3) / 1e9
    load_gbps = payload * args.steps / (load_ms / 1e3) / 1e9

    # ---- byte-exactness of what was just timed (untimed) -------------------
    checker = ByteChecker(torch, np, runtime, stream, w, src_cache, dst_cache, save_ids, load_ids,
                          payload_per_layer, page, offsets)
    checker.image(pool, "timed steps")
    checker.destination("timed steps")

    # ---- link peak: one large contiguous pinned <-> device copy -----------
    link_bytes = min(1 << 30, payload)
    scratch = torch.empty(link_bytes, device=dev, dtype=torch.uint8)

    def time_copy(fn, reps=5):
        fn()
        stream.synchronize()
        ev[0].record(stream)
        for _ in range(reps):
            fn()
        ev[1].record(stream)
        ev[1].synchronize()
        return link_bytes * reps / (ev[0].elapsed_ms(ev[1]) / 1e3) / 1e9

    d2h_peak = time_copy(lambda: runtime.memcpy_d2h_async(pool.host_ptr, scratch.data_ptr(),
                                                          link_bytes, stream))
    h2d_peak = time_copy(lambda: runtime.memcpy_h2d_async(scratch.data_ptr(), pool.host_ptr,
                                                          link_bytes, stream))
    # Restore what the link test overwrote in the pool.
    xfer.save(save_layers, stream, path)
    stream.synchronize()

    # ---- HBM copy ceiling with the same tile shape -------------------------
    scratch2 = torch.empty(link_bytes, device=dev, dtype=torch.uint8)
    lib = _lib.load()

    def plain():
        # tile_unroll 0: the same one-tile-per-workgroup form as the staged kernels
        _lib.check(lib.pf_plain_copy(scratch2.data_ptr(), scratch.data_ptr(), link_bytes, 0,
                                     stream.handle))
    hbm_copy_gbps = 2 * time_copy(plain, reps=20)

    # The same yardstick over the memory the gather and the scatter touch: plain
    # copies from the head of each layer's cache into a staging-sized buffer, and
    # back into each destination cache -- what the kernels would do if the block
    # ids were 0..n-1 and the layout one segment.  Measured the way the kernels'
    # `launches_alone` are: every launch between a pair of events of its own (so
    # the bracket is inside both figures), and of the size of a mean staged launch
    # of this workload (a layer's cache at most).  Copying one buffer pair over
    # and over (above) is placement-dependent and comes out faster than a walk
    # over 32 different caches.
    staged_launches_per_direction = max(live_launches_per_step // 2, 1)
    plain_launch_bytes = min(payload // staged_launches_per_direction, layer_bytes, link_bytes) & ~15
    plain_pairs = [(Event(timing=True), Event(timing=True)) for _ in range(3 * n_layers)]

    def plain_over_layers(to_cache):
        def once(pairs):
            for li in range(n_layers):
                cache = (dst_cache if to_cache else src_cache)[li].data_ptr()
                a, b = (cache, scratch.data_ptr()) if to_cache else (scratch.data_ptr(), cache)
                if pairs:
                    pairs[li][0].record(stream)
                _lib.check(lib.pf_plain_copy(a, b, plain_launch_bytes, 0, stream.handle))
                if pairs:
                    pairs[li][1].record(stream)
        once(None)
        stream.synchronize()
        for rep in range(3):
            once(plain_pairs[rep * n_layers: (rep + 1) * n_layers])
        stream.synchronize()
        total_ms = sum(a.elapsed_ms(b) for a, b in plain_pairs)
        return 2 * plain_launch_bytes * len(plain_pairs) / (total_ms / 1e3) / 1e9
    plain_gather_form = plain_over_layers(False)
    plain_scatter_form = plain_over_layers(True)

    # ---- roofline of the dominant kernel ------------------------------------
    # `achieved` comes from the events around every launch of the timed steps
    # (above).  A second, untimed pass times the launches running alone (the link
    # copies share the kernels' stream in that mode) and splits them by direction.
    xfer.set_kernel_timing(1)
    xfer.save(save_layers, stream, path)
    stream.synchronize()
    k_save_ms, k_save_n = xfer.last_kernel_ms()
    xfer.load(load_layers, stream, path)
    stream.synchronize()
    k_load_ms, k_load_n = xfer.last_kernel_ms()
    xfer.set_kernel_timing(0)
    alone_launches = k_save_n + k_load_n
    alone_launch_ms = (k_save_ms + k_load_ms) / max(alone_launches, 1)
    launches = live_launches_per_step
    assert launches == alone_launches, (launches, alone_launches)
    bytes_per_launch = 2 * payload / max(launches, 1)          # payload bytes one launch moves
    # staged: every payload byte is read once and written once in HBM -> 2 x
    # payload algorithmic bytes per launch; zero-copy: the kernel touches HBM
    # once per payload byte and is bounded by the host link, not by HBM
    staged_path = used_path == "staged"
    alg_bytes = (2 if staged_path else 1) * bytes_per_launch
    achieved = alg_bytes / (live_launch_ms / 1e3) / 1e9
    traffic, traffic_source = (measured_traffic(workload, alg_bytes) if staged_path
                               else (None, "zero-copy launches are not profiled for HBM traffic"))
    # What a pair of events reads with nothing between them on that stream: the
    # part of avg_launch_us that is the bracket itself, not the kernel (reported,
    # not subtracted).
    pair = [Event(timing=True), Event(timing=True)]
    empty_pair_us = []
    for _ in range(50):
        pair[0].record(stream)
        pair[1].record(stream)
        pair[1].synchronize()
        empty_pair_us.append(pair[0].elapsed_ms(pair[1]) * 1e3)
    empty_pair_us.sort()
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4),
                "traffic": traffic, "traffic_source": traffic_source,
                "kernel": ("block_tiles_rows_kernel / block_tiles_kernel (staged gather/scatter)" if staged_path
                           else "block_units_kernel (zero-copy, host-link bound)"),
                "measured": f"HIP events around each of the {live['launches']} launches of the "
                            f"{args.steps} timed steps",
                "launches": launches, "avg_launch_us": round(live_launch_ms * 1e3, 2),
                "empty_event_pair_us": round(empty_pair_us[len(empty_pair_us) // 2], 2),
                "alg_bytes_per_launch": int(alg_bytes),
                "launches_alone": {
                    "avg_launch_us": round(alone_launch_ms * 1e3, 2),
                    "achieved": round(alg_bytes / (alone_launch_ms / 1e3) / 1e9, 1),
                    "save_kernel_gbps": round(alg_bytes * k_save_n / (k_save_ms / 1e3) / 1e9, 1),
                    "load_kernel_gbps": round(alg_bytes * k_load_n / (k_load_ms / 1e3) / 1e9, 1)},
                "plain_copy_same_tile_gbps": round(hbm_copy_gbps, 1)}
    if staged_path:
        roofline["plain_copy_over_layers_gbps"] = {"from_caches": round(plain_gather_form, 1),
                                                   "into_caches": round(plain_scatter_form, 1),
                                                   "bytes_per_launch": 2 * plain_launch_bytes}
        # the launches that ran alone against the id-less copy of the same memory
        alone = roofline["launches_alone"]
        roofline["frac_of_plain_copy_over_layers"] = {
            "gather": round(alone["save_kernel_gbps"] / plain_gather_form, 3),
            "scatter": round(alone["load_kernel_gbps"] / plain_scatter_form, 3)}

    link = {"bound": "pcie_gen5_x16", "theoretical_gbps": PCIE_GEN5_X16_GBPS,
            "measured_d2h_gbps": round(d2h_peak, 2), "measured_h2d_gbps": round(h2d_peak, 2),
            "save_gbps": round(save_gbps, 2), "load_gbps": round(load_gbps, 2),
            "save_frac_of_measured": round(save_gbps / d2h_peak, 4),
            "load_frac_of_measured": round(load_gbps / h2d_peak, 4),
            "save_frac_of_theoretical": round(save_gbps / PCIE_GEN5_X16_GBPS, 4),
            "load_frac_of_theoretical": round(load_gbps / PCIE_GEN5_X16_GBPS, 4)}

    # The resource that bounds the step is the host link: payload bytes cross it
    # once, so achieved = payload / time against PCIe Gen5 x16, with the box's
    # measured one-large-copy rate beside the theoretical peak.
    link_t = (save_ms + load_ms) / 1e3
    link_achieved = 2 * payload * args.steps / link_t / 1e9
    link_measured = 2.0 / (1.0 / d2h_peak + 1.0 / h2d_peak)   # same bytes each way
    roofline["link"] = {"bound": "pcie_gen5_x16", "achieved": round(link_achieved, 2),
                        "peak": PCIE_GEN5_X16_GBPS, "unit": "GB/s",
                        "frac": round(link_achieved / PCIE_GEN5_X16_GBPS, 4),
                        "measured_peak": round(link_measured, 2),
                        "frac_of_measured": round(link_achieved / link_measured, 4),
                        "alg_bytes_per_step": 2 * payload,
                        "measured": "stream events around the save pass and the load pass of "
                                    "every timed step; measured_peak = one 1 GiB hipMemcpyAsync "
                                    "each way in this run (harmonic mean of d2h and h2d)"}

    # ---- compute overlap (configs[2]): transfers next to a GEMM stream ----
    overlap = None
    if "overlap" in sections:
        overlap = run_overlap(torch, xfer, save_layers, load_layers, stream, path, payload, n_layers,
                              checker, pool, m=args.gemm_m)

    # ---- both directions at once (the worker pool runs a load thread and a
    # save thread per GPU: gpu_worker.rs:116-345 of the reference) ----------
    duplex = None
    if "duplex" in sections:
        pool2 = PinnedMemory(payload)
        duplex = run_duplex(layers_for(src_cache, save_ids, pool2), load_layers, path, payload, args,
                            checker, pool, pool2, runtime)
        pool2.close()

    # ---- the same workload through the save / query / load engine -----------
    # In a process of its own, as the engine is deployed (a server that runs
    # nothing else on the GPU): which link copies the runtime overlaps depends
    # on the history of a process's streams, and this process has used many by
    # now.  The child allocates its own caches, so this one releases its first.
    byte_checks = list(checker.checked)
    del checker
    xfer.close()
    stream.close()
    pool.close()
    engine = None
    del src_cache, dst_cache, save_layers, load_layers, scratch, scratch2
    gc.collect()
    torch.cuda.empty_cache()
    # caches, the two 1 GiB yardstick buffers, staging and what the checker held
    released = 2 * n_layers * layer_bytes + 2 * link_bytes + (2 << 30)
    if "engine" in sections:
        import subprocess
        engine_pause = pause_after_free(runtime, released)
        def engine_run(mode, side_streams=False):
            cmd = [sys.executable, os.path.abspath(__file__), "--engine-child", "--workload",
                   workload, "--seed", str(args.seed), "--engine-mode", mode]
            if side_streams or args.engine_side_streams:
                cmd.append("--engine-side-streams")
            if args.engine_descriptors:
                cmd.append("--engine-descriptors")
            if args.engine_lazy_staging:
                cmd.append("--engine-lazy-staging")
            if args.layers:
                cmd += ["--layers", str(args.layers)]
            proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
            lines = [ln for ln in proc.stdout.splitlines() if ln.startswith("{")]
            if proc.returncode != 0 or not lines:
                print("bench.py: engine section failed:\n" + proc.stderr[-2000:], file=sys.stderr)
                sys.exit(1)
            return json.loads(lines[-1])
        engine = engine_run(args.engine_mode)
        engine["pause_before"] = engine_pause
        # the first child released its own caches and staging when it ended
        other_pause = pause_after_free(runtime, released + (4 << 30))
        # the other transfer mode, for comparison (instances choose one at registration)
        # the zero-copy worker mode, for comparison (instances choose a mode at registration;
        # "direct" and "kernel" both let the engine pick the path per call)
        other = "zerocopy" if args.engine_mode != "zerocopy" else "direct"
        engine["other_mode"] = engine_run(other)
        engine["other_mode"]["pause_before"] = other_pause
        released += 4 << 30
        # The opt-in form of the staged workers: link copies on a second stream per
        # worker (pf_engine_config.side_copy_streams), for comparison.
        if not args.engine_side_streams and args.engine_mode != "zerocopy":
            side_pause = pause_after_free(runtime, released)
            side = engine_run(args.engine_mode, side_streams=True)
            engine["side_copy_streams"] = {
                k: side.get(k) for k in ("save_gbps", "load_gbps", "save_gbps_first",
                                         "load_gbps_first", "save_gbps_all", "load_gbps_all",
                                         "concurrent_save_and_load", "staging_mib")}
            engine["side_copy_streams"]["pause_before"] = side_pause
            released += 4 << 30

    # ---- CPU baseline: the oracle's memcpy executor on the host cores -----
    cpu = None
    if "cpu" in sections:
        cpu = run_cpu_baseline(np, w, save_ids, load_ids, args.cpu_seconds, args.seed)

    result = {
        "metric": "KV save/load GB/s (GPU<->pinned host) & % of link peak, Llama-3.1-8B shape",
        "value": round(value, 3),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall * 1e3 / args.steps, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": f"{w['label']}, {n_layers} layers, {n} blocks saved then loaded "
                               "per step",
                   "layers": n_layers, "blocks": n, "fragment_bytes": seg,
                   "payload_bytes_per_direction": payload, "path": used_path,
                   "host_layout": "page-first" if w["page_first"] else "layer-first",
                   "staging_slot_mb": args.slot_mb or 512, "staging_slots": args.slots or 2,
                   "copy_stream": args.copy_stream},
        "save_gbps": round(save_gbps, 3),
        "step_save_load_ms": step_times[:16],
        "settle_steps": settle_steps,
        "link_at_start": link_at_start,
        "load_gbps": round(load_gbps, 3),
        "roofline": roofline,
        "link": link,
        "cpu_baseline": cpu,
        "overlap": overlap,
        "duplex": duplex,
        "engine": engine,
        "byte_checks": byte_checks,
        "verified": True,   # a failed byte check ends the run with exit status 1
        "device_bytes_released": released,
        "pool_alloc_s": round(pool_alloc_s, 2),
        "device": runtime.device_name(0),
    }
    return result


class ByteChecker:
    """Byte checks of what the bench moves, on every layer: the host image holds
    block save_ids[i] of the source cache at list position i (K buffer then V
    buffer per layer, or one page per block with the layers at their offsets),
    and the destination cache holds it at block load_ids[i] with every other
    block still zero.  The comparisons run on the device (the image is uploaded
    a piece at a time); a difference ends the bench with exit status 1."""

    PAGES_PER_PIECE = 128

    def __init__(self, torch, np, runtime, stream, w, src, dst, save_ids, load_ids,
                 payload_per_layer, page, offsets):
        self.torch, self.runtime, self.stream = torch, runtime, stream
        self.src, self.dst = src, dst
        self.nb, self.seg, self.n = w["num_blocks"], w["seg"], w["n"]
        self.nseg = 2 if w["split"] else 1
        self.page_first, self.page, self.offsets = w["page_first"], page, offsets
        self.payload_per_layer = payload_per_layer
        dev = src[0].device
        self.sid = torch.from_numpy(save_ids.astype(np.int64)).to(dev)
        self.lid = torch.from_numpy(load_ids.astype(np.int64)).to(dev)
        untouched = torch.ones(self.nb, dtype=torch.bool, device=dev)
        untouched[self.lid] = False
        self.rest = torch.nonzero(untouched).reshape(-1)
        piece = self.PAGES_PER_PIECE * page if self.page_first else payload_per_layer
        self.piece = torch.empty(piece, device=dev, dtype=torch.uint8)
        self.zeros = torch.zeros(piece, device=dev, dtype=torch.uint8)
        self.checked = []

    def _fail(self, message):
        print("bench.py: byte check failed: " + message, file=sys.stderr)
        sys.exit(1)

    def _pieces(self, total):
        step = self.piece.numel()
        return [(o, min(step, total - o)) for o in range(0, total, step)]

    def clear_image(self, pool):
        total = self.n * self.page if self.page_first else self.payload_per_layer * len(self.src)
        for off, size in self._pieces(total):
            self.runtime.memcpy_d2h_async(pool.host_ptr + off, self.zeros.data_ptr(), size, self.stream)
        self.stream.synchronize()

    def clear_destination(self):
        for t in self.dst:
            t.zero_()
        self.torch.cuda.synchronize()

    def _upload(self, pool, off, size):
        self.runtime.memcpy_h2d_async(self.piece.data_ptr(), pool.host_ptr + off, size, self.stream)
        self.stream.synchronize()

    def image(self, pool, what):
        torch = self.torch
        if self.page_first:
            for off, size in self._pieces(self.n * self.page):
                self._upload(pool, off, size)
                first, k = off // self.page, size // self.page
                got = self.piece[:size].view(k, self.page)
                for li, cache in enumerate(self.src):
                    want = cache.view(torch.uint8).view(self.nb, self.seg)[self.sid[first:first + k]]
                    lo = self.offsets[li]
                    if not torch.equal(got[:, lo:lo + self.seg], want):
                        self._fail(f"{what}: host pages {first}..{first + k - 1}, layer {li}")
        else:
            for li, cache in enumerate(self.src):
                self._upload(pool, li * self.payload_per_layer, self.payload_per_layer)
                want = cache.view(torch.uint8).view(self.nseg, self.nb, self.seg)[:, self.sid]
                if not torch.equal(self.piece.view(self.nseg, self.n, self.seg), want):
                    self._fail(f"{what}: host image of layer {li} differs from the device cache")
        self.checked.append(f"{what}: host image, {len(self.src)} layers")

    def destination(self, what):
        torch = self.torch
        for li, (s_, d_) in enumerate(zip(self.src, self.dst)):
            s_ = s_.view(torch.uint8).view(self.nseg, self.nb, self.seg)
            d_ = d_.view(torch.uint8).view(self.nseg, self.nb, self.seg)
            if not torch.equal(d_[:, self.lid], s_[:, self.sid]):
                self._fail(f"{what}: layer {li}: loaded blocks differ")
            if bool(d_[:, self.rest].any()):
                self._fail(f"{what}: layer {li}: a block outside the list changed")
        self.checked.append(f"{what}: destination cache, {len(self.dst)} layers")


def run_overlap(torch, xfer, save_layers, load_layers, stream, path, payload, n_layers, checker,
                pool, m=4096):
    """Transfer alone, GEMM stream alone, then both at once (load and save).
    The pass that runs next to the GEMM stream starts from a cleared target and
    is byte-checked on every layer; the GEMM's result is compared with the one
    it gives alone."""
    from pegaflow_amd.runtime import Event, Stream
    dev = torch.device("cuda:0")
    a = torch.randn(m, m, device=dev, dtype=torch.bfloat16)
    b = torch.randn(m, m, device=dev, dtype=torch.bfloat16)
    c = torch.empty(m, m, device=dev, dtype=torch.bfloat16)
    gemm_stream = torch.cuda.Stream()
    flop = 2.0 * m * m * m
    g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0, e1 = Event(timing=True), Event(timing=True)
    layer_ev = [Event(timing=True) for _ in range(n_layers)]

    ticks = []   # (GEMMs launched so far, event on the GEMM stream), one per 64 GEMMs

    def gemms(count, tick_pool=None, until=None, start=0):
        """Launch `count` GEMMs; with `until` (an event on another stream), keep
        launching in groups of 64 after that until the event has completed, so
        that the GEMM stream stays busy for as long as that work takes.  `start`
        continues the numbering (and the marks) of an earlier call.
        Returns the number launched by this call."""
        if start == 0:
            del ticks[:]
        launched = start
        first = True
        with torch.cuda.stream(gemm_stream):
            g0.record()
            while True:
                for _ in range(count if first else 64):
                    torch.matmul(a, b, out=c)
                    launched += 1
                    if tick_pool is not None and launched % 64 == 0 and launched // 64 <= len(tick_pool):
                        tick_pool[launched // 64 - 1].record(gemm_native)
                        ticks.append((launched, tick_pool[launched // 64 - 1]))
                first = False
                if until is None or until.query() or launched > 60000:
                    break
            g1.record()
        return launched - start

    gemms(50)
    torch.cuda.synchronize()
    gemms(200)
    torch.cuda.synchronize()
    gemm_alone_ms = g0.elapsed_time(g1) / 200
    gemm_native = Stream.wrap(gemm_stream.cuda_stream)
    m0, m1 = Event(timing=True), Event(timing=True)
    tick_pool = [Event(timing=True) for _ in range(1024)]
    c_alone = c.clone()
    out = {"gemm": f"{m}x{m}x{m} bf16, back to back on its own stream",
           "gemm_alone_tflops": round(flop / (gemm_alone_ms / 1e3) / 1e12, 1)}
    gemm_ok = True
    for name, fn, layers in (("load", xfer.load, load_layers), ("save", xfer.save, save_layers)):
        e0.record(stream)
        fn(layers, stream, path)
        e1.record(stream)
        e1.synchronize()
        alone_ms = e0.elapsed_ms(e1)
        if name == "load":
            xfer.set_layer_events(layer_ev)
            checker.clear_destination()
        else:
            checker.clear_image(pool)
        c.zero_()
        torch.cuda.synchronize()
        # A backlog of GEMMs, the transfer (the call only enqueues), then more GEMMs
        # until the transfer's end event has completed: the GEMM stream is busy
        # from before the transfer starts until after it ends.
        m0.record(gemm_native)
        backlog = gemms(960, tick_pool)           # 15 marks before and into the transfer
        e0.record(stream)
        fn(layers, stream, path)
        e1.record(stream)
        count = gemms(64, tick_pool, until=e1, start=backlog)  # those launched after the call
        m1.record(gemm_native)
        e1.synchronize()
        torch.cuda.synchronize()
        # share of the transfer during which the GEMM stream was running
        begin, end = m0.elapsed_ms(e0), m0.elapsed_ms(e1)
        together = (min(m0.elapsed_ms(m1), end) - max(0.0, begin)) / (end - begin)
        xfer.set_layer_events(None)
        both_ms = e0.elapsed_ms(e1)
        if name == "load":
            checker.destination("load next to the GEMM stream")
        else:
            checker.image(pool, "save next to the GEMM stream")
        gemm_ok = gemm_ok and bool(torch.equal(c, c_alone))
        # GEMM rate while the transfer was in flight: between the first and the last
        # of the marks (one per 64 GEMMs) that fell inside the transfer's span
        inside = [(k, m0.elapsed_ms(ev)) for k, ev in ticks]
        inside = [(k, t) for k, t in inside if begin <= t <= end]
        if len(inside) >= 2:
            during_ms = (inside[-1][1] - inside[0][1]) / (inside[-1][0] - inside[0][0])
            out[f"gemm_with_{name}_tflops"] = round(flop / (during_ms / 1e3) / 1e12, 1)
        else:
            # Fewer than two marks inside: the GEMM stream all but stood still.  The
            # GEMMs between the last mark before the transfer and the first after it
            # bound what it did meanwhile.
            out[f"gemm_with_{name}_tflops"] = None
            marks = [(k, m0.elapsed_ms(ev)) for k, ev in ticks]
            before = [m for m in marks if m[1] < begin]
            after = [m for m in marks if m[1] > end]
            if before and after:
                out[f"gemm_with_{name}_tflops_at_most"] = round(
                    flop * (after[0][0] - before[-1][0]) / ((end - begin) / 1e3) / 1e12, 1)
        out[f"gemm_stream_with_{name}_tflops_whole_run"] = round(
            flop / (g0.elapsed_time(g1) / count / 1e3) / 1e12, 1)
        out[f"{name}_alone_gbps"] = round(payload / (alone_ms / 1e3) / 1e9, 2)
        out[f"{name}_with_gemm_gbps"] = round(payload / (both_ms / 1e3) / 1e9, 2)
        out[f"{name}_share_next_to_gemm"] = round(together, 3)
        if name == "load":
            done = [e0.elapsed_ms(le) for le in layer_ev]
            per_layer = [done[0]] + [done[i] - done[i - 1] for i in range(1, len(done))]
            out["per_layer_ms_mean"] = round(sum(per_layer) / len(per_layer), 3)
            out["per_layer_ms_max"] = round(max(per_layer), 3)
            out["first_layer_ready_ms"] = round(done[0], 3)
    if not gemm_ok:
        print("bench.py: the GEMM next to a transfer differs from the GEMM alone", file=sys.stderr)
        sys.exit(1)
    out["verified"] = True
    out["verified_what"] = ("every layer of the destination caches (load) and of the host image (save) "
                            "after the passes that ran next to the GEMM stream; GEMM result equal to "
                            "the GEMM alone")
    return out


def run_ref_transfer_bench(torch, np, args):
    """The reference's transfer bench (pegaflow-core/benches/transfer_h2d.rs:23-33,
    62-109,301-339): 4 KiB fragments, device slots of 8 KiB, 1024..65536
    fragments, layouts contiguous / strided_device / shuffled (xorshift64
    Fisher-Yates), both directions, 3 warm-up and 20 timed iterations of
    submit + synchronise, GiB/s = bytes * iters / seconds / 2^30 -- through
    the two descriptor backends and, for comparison, the block-ID path."""
    from pegaflow_amd.layout import KVCacheLayout
    from pegaflow_amd.runtime import PinnedMemory, Stream
    from pegaflow_amd.transfer import (BlockTransfer, KernelBackend, LayerBlocks, MemcpyBackend,
                                       TransferPath, desc_array)
    seg, stride_factor, warmup, iters = 4096, 2, 3, 20
    counts = [args.ref_fragments] if args.ref_fragments else [1024, 4096, 16384, 65536]
    dev = torch.device("cuda:0")
    max_n = max(counts)
    device_buf = torch.full((max_n * seg * stride_factor,), 0xA5, device=dev, dtype=torch.uint8)
    host = PinnedMemory(max_n * seg)
    idx = np.arange(max_n * seg, dtype=np.uint64)
    host.as_numpy()[:] = ((idx * 31 + 7) & 0xFF).astype(np.uint8)
    torch.cuda.synchronize()
    stream = Stream()
    backends = {"direct": MemcpyBackend(), "kernel": KernelBackend()}
    xfer = BlockTransfer()

    def shuffle(n):
        mask, state = (1 << 64) - 1, 0x9E3779B97F4A7C15
        perm = list(range(n))
        for i in range(n - 1, 0, -1):
            state ^= (state << 13) & mask
            state ^= state >> 7
            state ^= (state << 17) & mask
            j = state % (i + 1)
            perm[i], perm[j] = perm[j], perm[i]
        return np.array(perm, dtype=np.uint64)

    def gib_s(fn, nbytes):
        for _ in range(warmup):
            fn()
            stream.synchronize()
        # The interpreter's cyclic collector is paused while timing, as timeit does:
        # with torch loaded one full collection takes about 40 ms, eight iterations
        # of the largest case, and it falls into the same cell on every run.
        gc.collect()
        gc.disable()
        try:
            t0 = time.perf_counter()
            for _ in range(iters):
                fn()
                stream.synchronize()
            seconds = time.perf_counter() - t0
        finally:
            gc.enable()
        return nbytes * iters / seconds / 2 ** 30

    rows = []
    for n in counts:
        pos = np.arange(n, dtype=np.uint64)
        layouts = {
            # device slot of list position i; the host side is always dense in list order
            "contiguous": pos,
            "strided_device": pos * stride_factor,
            "shuffled": shuffle(n) * stride_factor,
        }
        for lname, slot in layouts.items():
            descs = desc_array(device_buf.data_ptr() + slot * seg, host.host_ptr + pos * seg,
                               host.device_ptr + pos * seg, seg, 0, 1)
            # the same bytes by block id: a contiguous layout of 4 KiB blocks
            layout = KVCacheLayout(device_buf.data_ptr(), device_buf.numel(), max_n * stride_factor,
                                   seg, 0, 1)
            lb = [LayerBlocks(layout=layout, block_ids=slot.astype(np.uint32),
                              host=(host.host_ptr,), host_device=(host.device_ptr,),
                              host_len=(n * seg,), host_stride=seg)]
            row = {"fragments": n, "layout": lname}
            for bname, b in backends.items():
                row[f"{bname}_d2h"] = round(gib_s(lambda: b.d2h(descs, stream), n * seg), 2)
                row[f"{bname}_h2d"] = round(gib_s(lambda: b.h2d(descs, stream), n * seg), 2)
            row["block_ids_d2h"] = round(gib_s(lambda: xfer.save(lb, stream, TransferPath.AUTO),
                                               n * seg), 2)
            row["block_ids_h2d"] = round(gib_s(lambda: xfer.load(lb, stream, TransferPath.AUTO),
                                               n * seg), 2)
            rows.append(row)
            print("bench.py: " + json.dumps(row), file=sys.stderr, flush=True)
    # byte check of the last case (shuffled, 65536 fragments, after its final load)
    got = device_buf.view(max_n * stride_factor, seg)[torch.from_numpy(
        layouts["shuffled"].astype(np.int64)).to(dev)].cpu().numpy().reshape(-1)
    if not np.array_equal(got, host.as_numpy()[:max_n * seg]):
        print("bench.py: device bytes differ from the host image", file=sys.stderr)
        sys.exit(1)
    headline = next(r for r in rows if r["fragments"] == max_n and r["layout"] == "shuffled")
    # The same kind of call timed from C++ (no interpreter between the calls): small
    # block-ID transfers and the smallest row of the table above, with plain
    # hipMemcpyAsync of the same sizes beside them.
    native = None
    native_bin = os.path.join(ROOT, "tests", "native", "small_transfers")
    if os.path.exists(native_bin) and not args.ref_fragments:
        import subprocess
        for o in (xfer, stream, host):
            o.close()
        for b in backends.values():
            b.close()
        del device_buf
        torch.cuda.empty_cache()
        proc = subprocess.run([native_bin], capture_output=True, text=True, timeout=300)
        lines = [ln for ln in proc.stdout.splitlines() if ln.startswith("{")]
        if proc.returncode != 0 or not lines:
            print("bench.py: tests/native/small_transfers failed:\n" + proc.stderr[-2000:],
                  file=sys.stderr)
            sys.exit(1)
        native = json.loads(lines[-1])
    print(json.dumps({
        "metric": "descriptor backends at the shapes of the reference's transfer bench "
                  "(4 KiB fragments), GiB/s",
        "value": headline["kernel_h2d"], "unit": "GiB/s", "n_gpus": 1, "steps": iters,
        "warmup": warmup, "ms_per_step": None, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "u8", "data": "synthetic",
        "config": {"workload": "benches/transfer_h2d.rs shapes: 4 KiB fragments, "
                               f"{counts[0]}..{max_n} per batch, contiguous/strided/shuffled, "
                               f"value = kernel backend, shuffled, {max_n} fragments, H2D"},
        "table": rows, "native_small_transfers": native}))


def run_ref_cpu_path():
    """The engine's CPU path on long block lists: tests/native/cpu_path.cpp, a C++
    program over the C ABI with the groups and shapes of the reference's
    pegaflow-core/benches/cpu_path.rs:389-774 (block counts 128..32768 of 1 KiB,
    one layer or 61).  value = blocks per second through save + flush at 8192
    unique blocks of one layer."""
    import subprocess
    native_bin = os.path.join(ROOT, "tests", "native", "cpu_path")
    if not os.path.exists(native_bin):
        print(f"bench.py: {native_bin} is missing: make -C pegaflow_amd/csrc", file=sys.stderr)
        sys.exit(1)
    proc = subprocess.run([native_bin], capture_output=True, text=True, timeout=900)
    lines = [ln for ln in proc.stdout.splitlines() if ln.startswith("{")]
    if proc.returncode != 0 or not lines:
        print("bench.py: tests/native/cpu_path failed:\n" + proc.stdout[-2000:] + proc.stderr[-2000:],
              file=sys.stderr)
        sys.exit(1)
    rows = json.loads(lines[-1])["rows"]
    head = next(r for r in rows if r["group"] == "save_flush_unique" and r["case"] == "8192")
    print(json.dumps({
        "metric": "engine CPU path at the shapes of the reference's cpu_path bench, blocks/s "
                  "(save + flush, 8192 unique 1 KiB blocks, one layer)",
        "value": round(8192 / head["mean_us"] * 1e6, 1), "unit": "blocks/s", "n_gpus": 1,
        "steps": 10, "warmup": 3, "ms_per_step": round(head["mean_us"] / 1e3, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": "benches/cpu_path.rs groups: save_flush_unique, "
                               "save_flush_cpu_multilayer_61, save_flush_dtoh_multilayer_61, "
                               "save/load_transfer_fragmentation, query_prefetch_lease, "
                               "load_submit_wait"},
        "table": rows}))


def run_engine(torch, np, runtime, w, names, src_cache, dst_cache, save_ids, load_ids, payload,
               mode_name="direct", descriptors=False, lazy_staging=False, side_copy_streams=False):
    """End to end through pf_engine_*: registration, batch_save (host image
    allocation in the pinned pool, one worker task, block bookkeeping), prefix
    query, batch_load into a second instance of the same namespace.  Times are
    wall clock around the C calls with the arguments packed beforehand.  The
    first repetition is the first task each worker ever sees; `*_gbps` are
    medians, `*_gbps_first` and `*_gbps_all` are beside them, and every load
    carries its phase profile (pf_task_result)."""
    from pegaflow_amd.engine import LayerSave, LoadState, PackedSaves, PegaEngine
    from pegaflow_amd.transfer import TransferMode
    nb, seg, n = w["num_blocks"], w["seg"], w["n"]
    nseg = 2 if w["split"] else 1
    n_layers = len(names)
    eng = PegaEngine(pool_size=int(payload * 2.3) + (256 << 20),
                     use_descriptor_backends=descriptors, lazy_staging=lazy_staging,
                     side_copy_streams=side_copy_streams)
    kv = nb * seg if nseg == 2 else 0
    for inst, caches in (("bench-src", src_cache), ("bench-dst", dst_cache)):
        eng.register_context_layer_batch(
            inst, "bench", 0, 0, 0, 1, 1, names, [t.data_ptr() for t in caches],
            [nseg * nb * seg] * n_layers, [nb] * n_layers, [seg] * n_layers, [kv] * n_layers,
            [nseg] * n_layers,
            transfer_mode=(TransferMode.ZEROCOPY if mode_name == "zerocopy"
                           else TransferMode.from_name(mode_name)),
            page_first=w["page_first"])
    for t in dst_cache:
        t.zero_()
    torch.cuda.synchronize()
    out = {"transfer_mode": mode_name, "worker_form": "descriptors" if descriptors else "block ids",
           "link_before_first_task": link_check(runtime),
           "staging_mib_after_registration": eng.staging_bytes >> 20,
           "lazy_staging": bool(lazy_staging), "side_copy_streams": bool(side_copy_streams)}
    reps = 5
    save_s, load_s, query_s, load_profiles = [], [], [], []
    for rep in range(reps):
        hashes = [bytes([rep]) + int(i).to_bytes(4, "little") + bytes(27) for i in range(n)]
        packed = PackedSaves([LayerSave(nm, save_ids, hashes) for nm in names])
        t0 = time.perf_counter()
        eng.batch_save_kv_blocks("bench-src", 0, 0, 0, packed)
        save_s.append(time.perf_counter() - t0)
        t0 = time.perf_counter()
        hits, lease = eng.query_prefix("bench-dst", hashes)
        query_s.append(time.perf_counter() - t0)
        assert hits == n, f"engine query found {hits} of {n} blocks"
        state = LoadState()
        t0 = time.perf_counter()
        task = eng.batch_load_kv_blocks_multi_layer("bench-dst", 0, 0, [names], lease,
                                                    [load_ids.tolist()], state)
        res = task.wait()   # raises if the load failed
        load_s.append(time.perf_counter() - t0)
        assert res.done and state.get() == 1, "engine load did not complete"
        load_profiles.append({"paths": list(res.paths), "staged_groups": res.staged_groups,
                              "zero_copy_launches": res.zero_copy_launches,
                              "elapsed_ms": round(res.elapsed_ms, 2),
                              **{k: round(v, 2) for k, v in res.phases_ms.items()}})
        task.close()
        state.close()
        if rep == reps - 1:
            out["save_profile_ms"] = {k: round(v, 2) for k, v in eng.last_save_profile().items()
                                      if k != "bytes"}
        eng.evict_all()
    dev = src_cache[0].device
    sid = torch.from_numpy(save_ids.astype(np.int64)).to(dev)
    lid = torch.from_numpy(load_ids.astype(np.int64)).to(dev)
    for li in sorted({0, n_layers - 1}):
        s_ = src_cache[li].view(torch.uint8).reshape(nseg, nb, seg)
        d_ = dst_cache[li].view(torch.uint8).reshape(nseg, nb, seg)
        if not torch.equal(d_[:, lid], s_[:, sid]):
            print(f"bench.py: engine round trip differs on layer {li}", file=sys.stderr)
            sys.exit(1)
    # A save and a load at once (the pool's two workers), from two threads.
    import threading
    try:
        hashes_a = [b"A" + int(i).to_bytes(4, "little") + bytes(27) for i in range(n)]
        hashes_b = [b"B" + int(i).to_bytes(4, "little") + bytes(27) for i in range(n)]
        packed_a = PackedSaves([LayerSave(nm, save_ids, hashes_a) for nm in names])
        packed_b = PackedSaves([LayerSave(nm, save_ids, hashes_b) for nm in names])
        eng.batch_save_kv_blocks("bench-src", 0, 0, 0, packed_a)
        hits, lease = eng.query_prefix("bench-dst", hashes_a)
        times = {}

        def do_save():
            t0 = time.perf_counter()
            eng.batch_save_kv_blocks("bench-src", 0, 0, 0, packed_b)
            times["save"] = time.perf_counter() - t0

        def do_load():
            t0 = time.perf_counter()
            task = eng.batch_load_kv_blocks_multi_layer("bench-dst", 0, 0, [names], lease,
                                                        [load_ids.tolist()])
            task.wait()
            times["load"] = time.perf_counter() - t0
            task.close()

        threads = [threading.Thread(target=do_save), threading.Thread(target=do_load)]
        t0 = time.perf_counter()
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        span = time.perf_counter() - t0
        out["concurrent_save_and_load"] = {
            "save_gbps": round(payload / times["save"] / 1e9, 2),
            "load_gbps": round(payload / times["load"] / 1e9, 2),
            "aggregate_gbps": round(2 * payload / span / 1e9, 2)}
    except Exception as exc:  # pool too small for two images, etc.: report, do not fail the bench
        out["concurrent_save_and_load"] = {"error": str(exc)}
    median = lambda xs: sorted(xs)[len(xs) // 2]
    out["save_gbps"] = round(payload / median(save_s) / 1e9, 2)
    out["load_gbps"] = round(payload / median(load_s) / 1e9, 2)
    out["save_gbps_first"] = round(payload / save_s[0] / 1e9, 2)
    out["load_gbps_first"] = round(payload / load_s[0] / 1e9, 2)
    out["first_over_median"] = {"save": round(median(save_s) / save_s[0], 4),
                                "load": round(median(load_s) / load_s[0], 4)}
    out["save_gbps_all"] = [round(payload / t / 1e9, 2) for t in save_s]
    out["load_gbps_all"] = [round(payload / t / 1e9, 2) for t in load_s]
    out["load_profile_first"] = load_profiles[0]
    out["load_profile_median_rep"] = load_profiles[load_s.index(median(load_s))]
    out["staging_mib"] = eng.staging_bytes >> 20
    out["query_ms"] = round(median(query_s) * 1e3, 2)
    out["blocks"] = n
    if not w["page_first"]:
        out["small_tasks_beside_short_kernels"] = engine_beside_short_kernels(
            torch, eng, names, save_ids, n_layers * nseg * seg)
    eng.close()
    return out


def engine_beside_short_kernels(torch, eng, names, save_ids, bytes_per_block, blocks=64, m=2048,
                                seconds=0.8):
    """What the engine's small tasks cost kernels that run beside them: a stream of
    back-to-back m^3 bf16 GEMMs (23 us each at 2048) alone, then beside an unbroken
    loop of save -> query -> load of `blocks` blocks per layer through the engine
    (4 MiB per layer at the Llama shape).  The workers of a `direct` / `kernel`
    instance stage such a task, those of a `zerocopy` instance move it with the
    resident kernel; the bench line carries both."""
    import threading
    from pegaflow_amd.engine import LayerSave
    dev = torch.device("cuda:0")
    a = torch.randn(m, m, device=dev, dtype=torch.bfloat16)
    b = torch.randn(m, m, device=dev, dtype=torch.bfloat16)
    c = torch.empty(m, m, device=dev, dtype=torch.bfloat16)
    gemm_stream = torch.cuda.Stream()
    ids = [int(i) for i in save_ids[:blocks]]
    stop = threading.Event()
    moved = {"bytes": 0, "seconds": 0.0, "error": None}

    def mover():
        salt = 0
        t0 = time.perf_counter()
        try:
            while not stop.is_set():
                salt += 1
                hashes = [b"k" + salt.to_bytes(4, "little") + i.to_bytes(4, "little") + bytes(23)
                          for i in range(len(ids))]
                eng.batch_save_kv_blocks("bench-src", 0, 0, 0,
                                         [LayerSave(nm, ids, hashes) for nm in names])
                hits, lease = eng.query_prefix("bench-dst", hashes)
                task = eng.batch_load_kv_blocks_multi_layer("bench-dst", 0, 0, [names], lease, [ids])
                task.wait()
                task.close()
                moved["bytes"] += 2 * len(ids) * bytes_per_block
                if salt % 64 == 0:
                    eng.evict_all()
        except Exception as exc:  # reported, the bench goes on
            moved["error"] = str(exc)
        moved["seconds"] = time.perf_counter() - t0

    def gemm_tflops(span):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        count = 0
        with torch.cuda.stream(gemm_stream):
            e0.record()
            t0 = time.perf_counter()
            while time.perf_counter() - t0 < span:
                for _ in range(256):
                    torch.matmul(a, b, out=c)
                count += 256
                if count % 4096 == 0:
                    gemm_stream.synchronize()   # keep the backlog bounded
            e1.record()
        e1.synchronize()
        return 2.0 * m ** 3 * count / (e0.elapsed_time(e1) / 1e3) / 1e12

    gemm_tflops(0.2)
    alone = gemm_tflops(seconds)
    thread = threading.Thread(target=mover)
    thread.start()
    time.sleep(0.1)
    beside = gemm_tflops(seconds)
    stop.set()
    thread.join()
    eng.evict_all()
    out = {"gemm": f"{m}x{m}x{m} bf16", "blocks_per_layer": len(ids),
           "task_mib": round(len(ids) * bytes_per_block / 2 ** 20, 1),
           "gemm_alone_tflops": round(alone, 1), "gemm_beside_tflops": round(beside, 1),
           "gemm_share_kept": round(beside / alone, 3),
           "engine_save_plus_load_gbps": round(moved["bytes"] / max(moved["seconds"], 1e-9) / 1e9, 2)}
    if moved["error"]:
        out["error"] = moved["error"]
    return out


def run_duplex(save_layers2, load_layers, path, payload, args, checker, pool, pool2, runtime):
    """A save and a load in flight together, each with its own stream and
    engine, as the two worker threads of one GPU issue them: the load scatters
    the host image of `pool` while the save gathers the same source blocks into
    a second pool.  Two forms: link copies on each engine's side stream (the
    stand-alone default) and on the callers' streams (what the worker pool
    configures).  `plain_pair_gbps` is the yardstick: two plain hipMemcpyAsync
    streams, 1 GiB copies, one stream per direction, in this same run.  The last
    pass of each form starts from cleared targets and is byte-checked."""
    from pegaflow_amd.runtime import Event, Stream
    from pegaflow_amd.transfer import BlockTransfer
    out = {}
    ev = [Event(timing=True) for _ in range(4)]

    # -- yardstick: plain copies, both directions at once --------------------
    piece = min(1 << 30, payload // 2)
    dbuf = checker.torch.empty(2 * piece, device=checker.src[0].device, dtype=checker.torch.uint8)
    sa, sb = Stream(), Stream()

    def pair(reps):
        ev[0].record(sa)
        ev[2].record(sb)
        for _ in range(reps):
            runtime.memcpy_d2h_async(pool2.host_ptr, dbuf.data_ptr(), piece, sa)
            runtime.memcpy_h2d_async(dbuf.data_ptr() + piece, pool2.host_ptr + piece, piece, sb)
        ev[1].record(sa)
        ev[3].record(sb)
        ev[1].synchronize()
        ev[3].synchronize()
        span = max(ev[0].elapsed_ms(ev[1]), ev[0].elapsed_ms(ev[3])) - min(0.0, ev[0].elapsed_ms(ev[2]))
        return {"d2h_gbps": round(piece * reps / ev[0].elapsed_ms(ev[1]) / 1e6, 2),
                "h2d_gbps": round(piece * reps / ev[2].elapsed_ms(ev[3]) / 1e6, 2),
                "aggregate_gbps": round(2 * piece * reps / span / 1e6, 2)}
    pair(1)
    out["plain_pair"] = pair(5)
    out["plain_pair_gbps"] = out["plain_pair"]["aggregate_gbps"]
    sa.close()
    sb.close()
    del dbuf

    for label, mode in (("side_stream_copies", 1), ("in_order_copies", 2)):
        xa, xb = (BlockTransfer(staging_slot_bytes=args.slot_mb << 20, staging_slots=args.slots,
                                tile_unroll=args.unroll, zerocopy_max_workgroups=args.zc_max_wg,
                                copy_stream=mode) for _ in range(2))
        sa, sb = Stream(), Stream()
        xa.save(save_layers2, sa, path)   # allocate staging
        xb.load(load_layers, sb, path)
        sa.synchronize()
        sb.synchronize()
        for rep in range(2):
            if rep == 1:
                checker.clear_image(pool2)
                checker.clear_destination()
            ev[0].record(sa)
            ev[2].record(sb)
            xa.save(save_layers2, sa, path)
            xb.load(load_layers, sb, path)
            ev[1].record(sa)
            ev[3].record(sb)
            ev[1].synchronize()
            ev[3].synchronize()
            save_ms, load_ms = ev[0].elapsed_ms(ev[1]), ev[2].elapsed_ms(ev[3])
            span_ms = max(ev[0].elapsed_ms(ev[1]), ev[0].elapsed_ms(ev[3]))
            out[label] = {"save_gbps": round(payload / save_ms / 1e6, 2),
                          "load_gbps": round(payload / load_ms / 1e6, 2),
                          "aggregate_gbps": round(2 * payload / span_ms / 1e6, 2),
                          "frac_of_plain_pair": round(2 * payload / span_ms / 1e6 /
                                                      out["plain_pair_gbps"], 4)}
        checker.image(pool2, f"save next to a load ({label})")
        checker.image(pool, f"image read by the load ({label})")
        checker.destination(f"load next to a save ({label})")
        for o in (xa, xb, sa, sb):
            o.close()
    out["verified"] = True
    return out


def run_cpu_baseline(np, w, save_ids, load_ids, seconds, seed):
    """Same workload shape, host cores only: one layer's cache resident in
    host memory, gathered into a host pool and scattered back with the
    oracle's memcpy-per-descriptor executor (a restatement of the reference's
    build_copy_descs -> one copy per descriptor), static chunks over threads.
    Sample: repeated save+load of one layer until `seconds` elapse."""
    from oracle import oracle as O
    threads = min(16, os.cpu_count() or 1)
    nb, seg, n = w["num_blocks"], w["seg"], w["n"]
    nseg = 2 if w["split"] else 1
    rng = np.random.default_rng(seed)
    cache = rng.integers(0, 256, size=nseg * nb * seg, dtype=np.uint8)
    dst = np.zeros_like(cache)
    host_k = np.zeros(n * seg, dtype=np.uint8)
    host_v = np.zeros(n * seg, dtype=np.uint8) if nseg == 2 else None
    kv = nb * seg if nseg == 2 else 0
    src_layout = O.layout_over(cache, nb, seg, kv, nseg)
    dst_layout = O.layout_over(dst, nb, seg, kv, nseg)

    def once(t):
        O.transfer_layer(src_layout, save_ids, host_k, host_v, host_is_src=False, threads=t)
        O.transfer_layer(dst_layout, load_ids, host_k, host_v, host_is_src=True, threads=t)

    once(threads)  # page in
    out = {}
    for label, t, budget in (("all", threads, seconds * 0.7), ("one", 1, seconds * 0.3)):
        reps, t0 = 0, time.perf_counter()
        while True:
            once(t)
            reps += 1
            el = time.perf_counter() - t0
            if el >= budget:
                break
        out[label] = 2 * nseg * n * seg * reps / el / 1e9
    # configs[0] verbatim (Qwen3-0.6B: 28 layers [2,2048,32768 B], 64 blocks
    # drawn per layer), gather into the pool then scatter back, all threads.
    q_layers, q_nb, q_n = 28, 2048, 64
    q_caches = [np.full(2 * q_nb * 32768, li + 1, dtype=np.uint8) for li in range(q_layers)]
    q_ids = [rng.choice(q_nb, q_n, replace=False).astype(np.uint32) for _ in range(q_layers)]
    q_layouts = [O.layout_over(c, q_nb, 32768, q_nb * 32768, 2) for c in q_caches]
    q_k = np.zeros(q_n * 32768, dtype=np.uint8)
    q_v = np.zeros(q_n * 32768, dtype=np.uint8)

    def qwen_pass():
        for lay, lid in zip(q_layouts, q_ids):
            O.transfer_layer(lay, lid, q_k, q_v, host_is_src=False, threads=threads)
            O.transfer_layer(lay, lid, q_k, q_v, host_is_src=True, threads=threads)

    qwen_pass()
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or time.perf_counter() - t0 < 1.0:
        qwen_pass()
        reps += 1
    q_gbps = 2 * q_layers * 2 * q_n * 32768 * reps / (time.perf_counter() - t0) / 1e9
    # A plain copy of 1 GiB in 4 MiB pieces over the same threads (a STREAM-copy
    # style yardstick for the host memory system; bytes counted once, as above).
    big_src = np.full(1 << 30, 7, dtype=np.uint8)
    big_dst = np.zeros(1 << 30, dtype=np.uint8)
    piece = 4 << 20
    rows = [(big_dst.ctypes.data + o, big_src.ctypes.data + o, big_src.ctypes.data + o, piece, 0, 0)
            for o in range(0, 1 << 30, piece)]
    O.exec_descs(rows, host_is_src=True, backend="kernel", threads=threads)
    reps, t0 = 0, time.perf_counter()
    while reps < 3 or time.perf_counter() - t0 < 1.0:
        O.exec_descs(rows, host_is_src=True, backend="kernel", threads=threads)
        reps += 1
    stream_gbps = (1 << 30) * reps / (time.perf_counter() - t0) / 1e9
    return {"value": round(out["all"], 2), "unit": "GB/s", "cores": threads, "kind": "port",
            "single_thread_gbps": round(out["one"], 2),
            "configs0_qwen3_0p6b_gbps": round(q_gbps, 2),
            "plain_copy_1gib_gbps": round(stream_gbps, 2),
            "sample": f"one layer [{nseg},{nb},{seg}B] host-resident, {n} blocks saved+loaded "
                      f"repeatedly for ~{seconds:.0f}s (oracle memcpy executor)"}


if __name__ == "__main__":
    main()
