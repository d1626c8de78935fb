/*
 * pegahip.h — C ABI of libpegahip.so: the MI355X (gfx950) implementation of
 * PegaFlow's layer-wise KV block transfer path.
 *
 * This is the boundary a `-sys` crate (or any FFI) binds in place of the CUDA
 * bindings the reference uses on this path.  Every entry point is `extern "C"`,
 * takes plain pointers and sizes, and cites the reference interface it stands
 * in for (paths are relative to the reference checkout).
 *
 * Conventions (reference: pegaflow-core/src/transfer/mod.rs:15-16,46-52):
 *  - Transfer calls only ENQUEUE onto the caller's stream and never synchronise.
 *    The caller keeps descriptors' device and host memory alive until it has
 *    synchronised the stream (or an event recorded after the call).
 *  - Return value: 0 = success; > 0 = a hipError_t from the HIP runtime;
 *    < 0 = one of the PF_ERR_* classes below.  After any non-zero return,
 *    pf_last_error() gives the message for the calling thread.
 *  - Handles are opaque pointers.  A backend / transfer handle belongs to one
 *    worker thread at a time (the reference's `TransferBackend: Send`, not
 *    `Sync`); pools and allocators are internally locked.
 *  - There is no CPU fallback: every call that moves bytes needs a HIP device
 *    and fails with a HIP error when none is present.
 */
#ifndef PEGAHIP_H
#define PEGAHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------ */
/* Status                                                                    */
/* ------------------------------------------------------------------------ */

/* Error classes; mirror `EngineError` (pegaflow-core/src/lib.rs, variants
 * InvalidArgument / Storage / CudaInit / WorkerMissing). */
#define PF_OK 0
#define PF_ERR_INVALID_ARGUMENT (-1)
#define PF_ERR_STORAGE (-2)
#define PF_ERR_DEVICE_INIT (-3)
#define PF_ERR_WORKER_MISSING (-4)
#define PF_ERR_INSTANCE_MISSING (-5)
#define PF_ERR_BUFFER_TOO_SMALL (-6)

/* Message of the last failing call on this thread ("" if none). */
const char* pf_last_error(void);
/* Library version string. */
const char* pf_version(void);

/* ------------------------------------------------------------------------ */
/* Device, stream, event                                                     */
/* Replaces cudarc CudaContext::new / new_stream / record_event /            */
/* event.synchronize (pegaflow-core/src/gpu_worker.rs:278-298,443-449).      */
/* ------------------------------------------------------------------------ */

typedef struct pf_stream_s* pf_stream_t; /* wraps a hipStream_t */
typedef struct pf_event_s* pf_event_t;   /* wraps a hipEvent_t */

int pf_device_count(int* out_count);
int pf_set_device(int device);
int pf_get_device(int* out_device);
int pf_device_synchronize(void);
/* NUMA node of the device from /sys/bus/pci/devices/<bdf>/numa_node; -1 when
 * unknown.  Replaces `nvidia-smi topo --get-numa-id-of-nearby-cpu`
 * (pegaflow-common/src/numa.rs:266-287). */
int pf_device_numa_node(int device, int* out_node);
int pf_device_name(int device, char* buf, size_t cap);

/* Non-blocking stream at the default priority. */
int pf_stream_create(pf_stream_t* out);
/* Wrap an existing hipStream_t (e.g. torch's) without owning it. */
int pf_stream_wrap(void* hip_stream, pf_stream_t* out);
int pf_stream_destroy(pf_stream_t s);
int pf_stream_synchronize(pf_stream_t s);
int pf_stream_wait_event(pf_stream_t s, pf_event_t e);
void* pf_stream_native(pf_stream_t s);
/* Do kernels of the two streams execute at the same time?  (The runtime
 * multiplexes a process's streams onto a few hardware queues; streams that
 * share one run their kernels strictly one after the other.)  *out = 1 when a
 * one-lane kernel on `a` saw, within 2 ms, a word posted by a one-lane kernel
 * on `b`.  Both streams are synchronised by the call.  The worker pools use
 * this when they are spawned (no counterpart in the reference, whose two worker
 * streams are never checked). */
int pf_streams_run_concurrently(pf_stream_t a, pf_stream_t b, int* out);

int pf_event_create(int enable_timing, pf_event_t* out);
int pf_event_destroy(pf_event_t e);
int pf_event_record(pf_event_t e, pf_stream_t s);
int pf_event_synchronize(pf_event_t e);
/* *out_done = 1 when complete, 0 when still pending. */
int pf_event_query(pf_event_t e, int* out_done);
int pf_event_elapsed_ms(pf_event_t start, pf_event_t stop, float* out_ms);

/* ------------------------------------------------------------------------ */
/* Pinned host memory                                                        */
/* Replaces PinnedMemory (pegaflow-core/src/pinned_mem.rs:100-397).          */
/* ------------------------------------------------------------------------ */

/* AllocStrategy, pinned_mem.rs:100-111. */
#define PF_HOST_REGULAR 0   /* mmap + parallel NUMA pre-touch + hipHostRegister(Mapped) */
#define PF_HOST_HIP_ALLOC 1 /* hipHostMalloc(Mapped); the default strategy */
#define PF_HOST_HUGEPAGES 2 /* mmap(MAP_HUGETLB) + pre-touch + hipHostRegister(Mapped) */

typedef struct pf_host_mem {
  void* host;          /* host virtual address */
  uint64_t device;     /* device-visible address of the same bytes */
  uint64_t size;       /* actual size (huge pages round up) */
  int32_t strategy;    /* PF_HOST_* */
  int32_t numa_node;   /* requested node, -1 = none */
} pf_host_mem;

/* numa_node < 0: placement follows the calling thread's affinity. */
int pf_host_alloc(uint64_t size, int strategy, int numa_node, pf_host_mem* out);
int pf_host_free(pf_host_mem* mem);
/* Worker count of the parallel pre-touch (pinned_mem.rs:368-376). */
uint64_t pf_touch_threads(uint64_t size);
/* Hugepagesize from /proc/meminfo in bytes, 0 when unavailable
 * (pinned_mem.rs:46-60). */
uint64_t pf_huge_page_size(void);

/* Device memory helpers for tests and benches; replace the reference's
 * test-only cuMemAlloc/cuMemcpy/cuMemset helpers
 * (pegaflow-core/tests/common/gpu_buffer.rs:13-69). */
int pf_dev_malloc(uint64_t size, uint64_t* out_ptr);
int pf_dev_free(uint64_t ptr);
int pf_dev_memset(uint64_t ptr, int value, uint64_t size);
int pf_dev_copy_from_host(uint64_t dst, const void* src, uint64_t size);
int pf_dev_copy_to_host(void* dst, uint64_t src, uint64_t size);
/* One contiguous async copy between device memory and pinned host memory on
 * `s`; the link-peak yardstick of the benches. */
int pf_memcpy_h2d_async(uint64_t dst, const void* src, uint64_t size, pf_stream_t s);
int pf_memcpy_d2h_async(void* dst, uint64_t src, uint64_t size, pf_stream_t s);

/* ------------------------------------------------------------------------ */
/* KV cache layout                                                           */
/* Replaces KVCacheLayout / BlockCopy / BlockCopies                          */
/* (pegaflow-core/src/layout.rs:13-286).                                     */
/* ------------------------------------------------------------------------ */

typedef struct pf_kv_layout {
  uint64_t data_ptr;             /* device base of this layer's cache */
  uint64_t size_bytes;           /* registered region size */
  uint64_t num_blocks;
  uint64_t block_stride_bytes;   /* step between consecutive blocks */
  uint64_t segment_bytes;        /* one of K or V (unpadded) */
  uint64_t segments;             /* 1, or 2 for K/V */
  uint64_t padded_segment_bytes; /* host-side stride of one segment */
  uint64_t kv_stride_bytes;      /* distance K -> V when split, else 0 */
  uint32_t split;                /* 1 = K and V in separate regions */
  uint32_t reserved;
} pf_kv_layout;

typedef struct pf_block_copy {
  uint64_t addr;
  uint64_t bytes;
} pf_block_copy;

/* KVCacheLayout::new, layout.rs:73-130. */
int pf_layout_new(uint64_t data_ptr, uint64_t size_bytes, uint64_t num_blocks,
                  uint64_t segment_bytes, uint64_t kv_stride_bytes,
                  uint64_t segments, pf_kv_layout* out);
/* KVCacheLayout::with_block_stride, layout.rs:140-153. */
int pf_layout_with_block_stride(pf_kv_layout* layout, uint64_t stride);
/* KVCacheLayout::with_ssd_padding, layout.rs:157-160. */
int pf_layout_with_ssd_padding(pf_kv_layout* layout, uint64_t alignment);
/* KVCacheLayout::block_copies, layout.rs:231-255: *out_n is 1 (contiguous) or
 * 2 (split: out[0] = K, out[1] = V). */
int pf_layout_block_copies(const pf_kv_layout* layout, uint64_t block_idx,
                           pf_block_copy out[2], uint32_t* out_n);
/* padded_block_bytes, layout.rs:283-285. */
uint64_t pf_layout_padded_block_bytes(const pf_kv_layout* layout);
/* block_bytes, layout.rs:271-273. */
uint64_t pf_layout_block_bytes(const pf_kv_layout* layout);

/* ------------------------------------------------------------------------ */
/* Copy descriptors and the two reference transfer backends                  */
/* Replaces CopyDesc / TransferBackend / TransferMode                        */
/* (pegaflow-core/src/transfer/mod.rs:36-76), MemcpyBackend                  */
/* (transfer/memcpy.rs:25-102) and KernelBackend (transfer/kernel.rs:25-135).*/
/* ------------------------------------------------------------------------ */

typedef struct pf_copy_desc {
  uint64_t device;            /* absolute device address */
  void* host;                 /* host virtual address */
  uint64_t host_device;       /* device-visible address of `host` */
  uint64_t size;
  uint64_t device_allocation; /* layer index */
  uint64_t host_allocation;   /* identity of the pinned allocation */
} pf_copy_desc;

typedef struct pf_merged_range {
  uint64_t device;
  void* host;
  uint64_t size;
} pf_merged_range;

/* As descriptor backends (pf_backend_create) the first two are the reference's:
 * "direct" issues DMA copies of the merged ranges, "kernel" one copy kernel
 * over mapped host memory.  As the mode of a worker pool or of an engine
 * registration they DEVIATE from the reference (gpu_worker.rs:264-276, where
 * Kernel selects the copy-kernel backend): both let the block-ID engine pick
 * the way across the link per task (PF_PATH_AUTO), because a copy kernel that
 * stays resident for a long transfer slows the model's kernels beside it; the
 * bytes moved are the same.  pf_task_result.paths says which way a task went,
 * the pool logs its choice once when it is spawned, and
 * pf_engine_config.kernel_mode_zerocopy gives PF_MODE_KERNEL registrations the
 * reference's behaviour. */
#define PF_MODE_DIRECT 0
#define PF_MODE_KERNEL 1
/* Worker pools and engine registrations only (not a descriptor backend, not a
 * name the connector sends): always the zero-copy kernel, whatever the size,
 * and no staging memory.  For instances that offload while the GPU is otherwise
 * idle; see pf_worker_pool_spawn. */
#define PF_MODE_ZEROCOPY 2

typedef struct pf_backend_s* pf_backend_t;

/* merge(), memcpy.rs:25-55.  `out` needs room for n entries. */
int pf_merge_copies(const pf_copy_desc* copies, uint64_t n, pf_merged_range* out,
                    uint64_t* out_n);
/* build_backend, gpu_worker.rs:264-276.  Binds to the current device. */
int pf_backend_create(int mode, pf_backend_t* out);
int pf_backend_destroy(pf_backend_t b);
/* TransferBackend::name: "direct" or "kernel". */
const char* pf_backend_name(pf_backend_t b);
/* TransferBackend::h2d / d2h.  Enqueue only.
 * Two things differ from the reference's MemcpyBackend, which issues one
 * stream-ordered copy per merged range in list order (memcpy.rs:57-102):
 *  - the "direct" backend reorders a batch (large ranges first, then isolated
 *    small ones, then packed runs), so a batch must not contain ranges whose
 *    DESTINATIONS overlap: which writer wins is not the list order;
 *  - a backend keeps internal staging shared by its batches.  Batches on one
 *    stream are ordered by the stream; a batch submitted on another stream
 *    waits (on the device) for the previous batch's use of the staging
 *    buffer.  A handle still belongs to one thread at a time. */
int pf_backend_h2d(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s);
int pf_backend_d2h(pf_backend_t b, const pf_copy_desc* copies, uint64_t n, pf_stream_t s);
/* The copy of PF_MODE_KERNEL for callers that cannot allocate: tight serving
 * loops, harnesses that forbid hipMalloc.  No counterpart in the reference (its
 * KernelBackend reallocates its device table whenever a batch outgrows it,
 * transfer/kernel.rs:102-111).  Same bytes as pf_backend_h2d (host_is_src != 0)
 * / pf_backend_d2h (host_is_src == 0) of a kernel backend, enqueue only, but the
 * device-side descriptor table lives in a fixed 1.5 MiB array inside the
 * library's device image and the call allocates no device or pinned memory
 * (no hipMalloc / hipFree / hipHostMalloc), on any call including the first.
 * Limits: n <= pf_desc_copy_noalloc_max() (32768), more is refused with
 * PF_ERR_INVALID_ARGUMENT; `copies` is read by the upload that the call
 * enqueues, so it stays alive and unchanged until the stream has been
 * synchronised (the usual descriptor rule), and it should sit in pinned memory
 * for that upload to be asynchronous (from pageable memory the runtime stages
 * it before the call returns); every call on one GPU shares the one table, so
 * the library orders them: a call waits, on the device, for the kernel of the
 * call before it, whatever streams the two use (calls on different streams of
 * one GPU do not overlap).  Not tested under HIP graph capture. */
int pf_desc_copy_noalloc(const pf_copy_desc* copies, uint64_t n, int host_is_src, pf_stream_t s);
uint64_t pf_desc_copy_noalloc_max(void);
/* TransferMode from the connector's string ("direct" | "kernel"),
 * python/pegaflow/connector/common.py:577-594. */
int pf_transfer_mode_from_name(const char* name, int* out_mode);

/* ------------------------------------------------------------------------ */
/* Descriptor construction from layouts x blocks                             */
/* Replaces build_copy_descs (pegaflow-core/src/gpu_worker.rs:353-423) and   */
/* the host-block view it reads (block.rs:62-199, gpu_worker.rs:63-94).      */
/* ------------------------------------------------------------------------ */

typedef struct pf_host_block {
  void* seg_host[2];       /* host address of segment 0 / 1 */
  uint64_t seg_device[2];  /* device-visible address of segment 0 / 1 */
  uint64_t seg_alloc[2];   /* allocation identity of segment 0 / 1 */
  uint64_t seg_size[2];    /* (padded) size of segment 0 / 1 */
  uint32_t num_segments;   /* 1 or 2 */
  uint32_t reserved;
  uint64_t host_offset;    /* page-first byte offset of this layer; else 0 */
} pf_host_block;

typedef struct pf_layer_transfer {
  const char* layer_name;
  pf_kv_layout layout;
  const uint64_t* block_idx;   /* device slot of each block */
  const pf_host_block* blocks; /* host image of each block */
  uint64_t n_blocks;
} pf_layer_transfer;

/* Writes up to `cap` descriptors; *out_n is the count needed.  Returns
 * PF_ERR_BUFFER_TOO_SMALL when cap < *out_n (nothing else is wrong). */
int pf_build_copy_descs(const pf_layer_transfer* layers, uint64_t n_layers,
                        pf_copy_desc* out, uint64_t cap, uint64_t* out_n,
                        uint64_t* out_total_bytes);

/* ------------------------------------------------------------------------ */
/* Block-ID gather / scatter (the MI355X fast path)                          */
/* Same bytes as build_copy_descs + TransferBackend::{d2h,h2d}               */
/* (gpu_worker.rs:353-423,441,494) with no per-fragment descriptor: the      */
/* kernels compute `data_ptr + id*block_stride (+ kv_stride)` themselves.    */
/* ------------------------------------------------------------------------ */

typedef struct pf_layer_blocks {
  const char* layer_name;    /* for error messages; may be NULL */
  pf_kv_layout layout;
  const uint32_t* block_ids; /* host array: device slot of block i */
  uint64_t n_blocks;
  /* Host image.  Segment s of block i lives at
   *   host[s] + i*host_stride                       (page_host == NULL), or
   *   page_host[i] + page_offset + s*segment_bytes  (page_host != NULL).
   * For a contiguous (non-split) layout only host[0] is used and one block
   * is one fragment of block_bytes. */
  void* host[2];
  uint64_t host_device[2];
  uint64_t host_len[2];         /* bytes available behind host[s] */
  uint64_t host_stride;
  const uint64_t* page_host;        /* optional per-block page bases (host VA) */
  const uint64_t* page_host_device; /* same, device-visible */
  uint64_t page_offset;
  uint64_t page_len;                /* bytes available behind each page base */
} pf_layer_blocks;

/* How bytes cross the host link. */
#define PF_PATH_AUTO 0     /* pick per shape */
#define PF_PATH_ZEROCOPY 1 /* kernel reads/writes mapped host memory */
#define PF_PATH_STAGED 2   /* device gather/scatter + one DMA copy per unit */

typedef struct pf_xfer_config {
  uint64_t staging_slot_bytes; /* 0 = default */
  uint32_t staging_slots;      /* 0 = default (2) */
  uint32_t zerocopy_max_workgroups; /* workgroups of a zero-copy launch; 0 = default (16 for
                                       fragments of 16 KiB and more, up to 64 for smaller ones) */
  uint64_t auto_staged_min_bytes;   /* PF_PATH_AUTO stages a dense layer of this size or more;
                                       0 = default (16 MiB) */
  uint32_t tile_unroll;             /* zero-copy kernel: 16-byte loads in flight per lane:
                                       1,2,4,8; 0 = default (4) */
  uint32_t copy_stream;             /* staged path: where the link copies run.
                                       0 = default (side stream when a call has more than
                                       one staged unit), 1 = a side stream of the engine (the
                                       copy of one unit overlaps the gather of the next),
                                       2 = the caller's stream (in order, no second queue) */
  uint64_t auto_staged_min_call_bytes; /* PF_PATH_AUTO also stages every dense layer (of 32 KiB or
                                       more) of a call whose dense layers add up to this much;
                                       0 = off.  For engines that move KV beside running kernels:
                                       the resident zero-copy kernel costs those for as long as
                                       the call lasts. */
  uint64_t staged_group_bytes;      /* staged layers that follow one another share one staging
                                       slot, and one gather / scatter launch, while together
                                       they stay below this size (and the slot's); a group's
                                       layers complete together.  0 = default: every slot is
                                       filled to the brim, a layer split where the slot ends,
                                       or whole layers up to 32 MiB while per-layer events
                                       are set (pf_xfer_set_layer_events). */
} pf_xfer_config;

typedef struct pf_xfer_s* pf_xfer_t;

int pf_xfer_create(const pf_xfer_config* cfg, pf_xfer_t* out);
int pf_xfer_destroy(pf_xfer_t x);
/* Save: gather the listed blocks of every layer into their host images. */
int pf_xfer_save(pf_xfer_t x, const pf_layer_blocks* layers, uint64_t n_layers,
                 int path, pf_stream_t s);
/* Load: scatter host images into the listed device slots. */
int pf_xfer_load(pf_xfer_t x, const pf_layer_blocks* layers, uint64_t n_layers,
                 int path, pf_stream_t s);
/* Optional per-layer completion events: when set (n >= n_layers of the next
 * call) each layer's event is recorded when that layer's bytes have landed.
 * Pass NULL to clear. */
int pf_xfer_set_layer_events(pf_xfer_t x, pf_event_t* events, uint64_t n);
/* Path the last call took for layer 0 (PF_PATH_ZEROCOPY or PF_PATH_STAGED). */
int pf_xfer_last_path(pf_xfer_t x);
/* Timing of the device-side gather/scatter kernels, measured with events on
 * the stream the kernels ran on: total milliseconds and launches.  Blocks until
 * those events have completed.  pf_xfer_set_kernel_timing: 0 = off; 1 = every
 * launch is timed running alone (the link copies of the staged path share the
 * kernels' stream while this is on) and the figures are those of the last call;
 * 2 = launches are timed where they run, streams unchanged, and the figures add
 * up over calls until pf_xfer_last_kernel_ms reads (and clears) them. */
int pf_xfer_last_kernel_ms(pf_xfer_t x, float* out_ms, uint32_t* out_launches);
int pf_xfer_set_kernel_timing(pf_xfer_t x, int enable);

/* How pf_xfer_save / pf_xfer_load cut the staged layers of one call into units
 * (runs of list positions of one layer) and pack the units into staging-slot
 * fills, one gather or scatter launch and its link copies per fill: the planner
 * those calls use, as pure host arithmetic (no device needed), for callers that
 * want to know what a call will cost and for tests.  layer_blocks[i] = list
 * positions of layer i, block_bytes[i] = payload bytes of one position (all
 * segments; 0 = the layer is not staged and gets one unit outside any fill).
 * slot_bytes and group_bytes as in pf_xfer_config (0 = default);
 * per_layer_events != 0 = as after pf_xfer_set_layer_events.  Writes at most
 * `capacity` units to `out` (may be NULL when capacity is 0) and always the
 * number of units and of fills.  No counterpart in the reference. */
typedef struct pf_fill_unit {
  uint64_t layer;       /* index into the call's layers */
  uint64_t first;       /* first list position of the unit */
  uint64_t count;       /* list positions */
  uint64_t slot_offset; /* byte offset of the unit inside its fill's staging slot */
  uint64_t fill;        /* number of the fill the unit belongs to; UINT64_MAX = not staged */
} pf_fill_unit;

int pf_plan_staged_fills(const uint64_t* layer_blocks, const uint64_t* block_bytes,
                         uint64_t n_layers, uint64_t slot_bytes, uint64_t group_bytes,
                         uint32_t per_layer_events, pf_fill_unit* out, uint64_t capacity,
                         uint64_t* out_units, uint64_t* out_fills);

/* Plain device-to-device copy with the same tile shape as the gather/scatter
 * kernels (pointers and size 16-byte aligned).  tile_unroll 0 = the
 * one-tile-per-workgroup form of the staged path; 1/2/4/8 = the grid-stride
 * form of the zero-copy path.  A copy of known size: the
 * yardstick for the HBM copy ceiling and for scaling hardware counters.  No
 * counterpart in the reference. */
int pf_plain_copy(uint64_t dst, uint64_t src, uint64_t bytes, uint32_t tile_unroll,
                  pf_stream_t s);

/* ------------------------------------------------------------------------ */
/* Offset allocator (pure host arithmetic)                                   */
/* Replaces ScaledOffsetAllocator (pegaflow-core/src/allocator.rs:63-142)    */
/* over the `offset-allocator` crate.                                        */
/* ------------------------------------------------------------------------ */

typedef struct pf_allocator_s* pf_allocator_t;

typedef struct pf_alloc_region {
  uint64_t offset_bytes;
  uint64_t size_bytes; /* rounded up to the unit; 0 = no space */
  uint64_t token;      /* pass back to pf_allocator_free */
} pf_alloc_region;

/* new_with_unit_size_and_max_allocs, allocator.rs:73-92. */
int pf_allocator_create(uint64_t total_bytes, uint64_t unit_size, uint32_t max_allocs,
                        pf_allocator_t* out);
int pf_allocator_destroy(pf_allocator_t a);
/* allocate, allocator.rs:95-123: PF_OK with size_bytes == 0 when nothing fits
 * (or size is 0); PF_ERR_INVALID_ARGUMENT when the request overflows u32 units. */
int pf_allocator_allocate(pf_allocator_t a, uint64_t size_bytes, pf_alloc_region* out);
int pf_allocator_free(pf_allocator_t a, const pf_alloc_region* region);
/* total_bytes + storage_report, allocator.rs:131-142. */
int pf_allocator_report(pf_allocator_t a, uint64_t* out_total_bytes, uint64_t* out_free_bytes,
                        uint64_t* out_largest_free_bytes, uint64_t* out_total_units);

/* ------------------------------------------------------------------------ */
/* Pinned pool                                                               */
/* Replaces PinnedAllocator / ShardedPinnedPool / NumaAwarePinnedPools /     */
/* PinnedMemoryPool / PinnedAllocation                                       */
/* (pegaflow-core/src/pinned_pool.rs:56-715).                                */
/* ------------------------------------------------------------------------ */

typedef struct pf_pool_s* pf_pool_t;

typedef struct pf_pool_config {
  uint64_t capacity;        /* total bytes, split evenly over NUMA nodes and shards */
  uint32_t num_shards;      /* per node; 0 or 1 = one pool */
  uint32_t use_hugepages;   /* MAP_HUGETLB backing */
  uint32_t ssd_enabled;     /* regular (CPU-readable) backing instead of hipHostMalloc */
  uint32_t n_numa_nodes;    /* 0 = one global pool */
  const int32_t* numa_nodes;
  uint64_t unit_size_hint;  /* 0 = 512 */
} pf_pool_config;

typedef struct pf_allocation {
  uint64_t handle;  /* owning handle; 0 when the pool is exhausted */
  void* host;
  uint64_t device;
  uint64_t size;    /* bytes actually reserved (unit-rounded) */
} pf_allocation;

/* compute_unit_size, pinned_pool.rs:135-141. */
uint64_t pf_pool_compute_unit_size(uint64_t pool_size, uint64_t unit_size_hint);
/* PinnedAllocator::new_global / new_numa, pinned_pool.rs:616-660. */
int pf_pool_create(const pf_pool_config* cfg, pf_pool_t* out);
int pf_pool_destroy(pf_pool_t p);
/* allocate, pinned_pool.rs:666-675.  numa_node is ignored by a global pool.
 * PF_OK with handle == 0 when nothing fits (the reference's `None`). */
int pf_pool_allocate(pf_pool_t p, uint64_t size, int numa_node, pf_allocation* out);
/* Drop of the PinnedAllocation guard, pinned_pool.rs:112-117. */
int pf_pool_free(pf_allocation* a);
int pf_pool_usage(pf_pool_t p, uint64_t* out_used, uint64_t* out_total);
int pf_pool_largest_free(pf_pool_t p, int numa_node, uint64_t* out_bytes);
int pf_pool_is_numa(pf_pool_t p);

/* ------------------------------------------------------------------------ */
/* NUMA helpers (pegaflow-common/src/numa.rs:49-257)                         */
/* ------------------------------------------------------------------------ */

/* format_cpu_list: [0,1,2,4] -> "0-2,4". */
int pf_numa_format_cpu_list(const uint64_t* cpus, uint64_t n, char* buf, size_t cap);
/* parse_cpulist: "0-3,8" -> sorted unique ids; *out_n = count needed. */
int pf_numa_parse_cpulist(const char* cpulist, uint64_t* out, uint64_t cap, uint64_t* out_n);
/* pin_thread_to_numa_node for the calling thread. */
int pf_numa_pin_thread(int numa_node);
/* Number of NUMA nodes with CPUs (1 when sysfs has none). */
int pf_numa_node_count(void);
/* NUMA node of a PCI device under `sysfs_root` (NULL = /sys/bus/pci/devices). */
int pf_numa_node_of_pci(const char* bdf, const char* sysfs_root);
/* query_pages_numa, numa.rs:448-476: the NUMA node each address currently
 * resides on (move_pages query), -1 where unknown. */
int pf_numa_query_pages(const void* const* addrs, uint64_t n, int* out_nodes);

/* ------------------------------------------------------------------------ */
/* Layer topology and page-first placement                                   */
/* Replaces build_page_layout / LayerTopology                                */
/* (pegaflow-core/src/instance.rs:46-269,488-672).                           */
/* ------------------------------------------------------------------------ */

/* build_page_layout, instance.rs:107-162.  Worker w registered the layer ids
 * set_ids[set_off[w] .. set_off[w+1]).  Outputs are indexed by layer id
 * (n_layers entries) and by shard (*out_n_shards <= n_sets entries). */
int pf_build_page_layout(const uint64_t* set_ids, const uint64_t* set_off, uint64_t n_sets,
                         uint64_t n_layers, const uint64_t* padded_bytes,
                         uint64_t* out_layer_shard, uint64_t* out_layer_offsets,
                         uint64_t* out_layer_bytes, uint64_t* out_shard_page_sizes,
                         uint64_t* out_n_shards);

typedef struct pf_topology_s* pf_topology_t;

typedef struct pf_worker_layers {
  int32_t device_id;
  uint32_t tp_rank;
  uint32_t pp_rank;
  uint32_t n_layers;
  const char* const* layer_names;
  const pf_kv_layout* layouts;
  const uint32_t* group_ids; /* NULL = all group 0 */
} pf_worker_layers;

/* seal_topology, instance.rs:488-672. */
int pf_topology_seal(const pf_worker_layers* workers, uint32_t n_workers, uint32_t tp_size,
                     int page_first, pf_topology_t* out);
int pf_topology_destroy(pf_topology_t t);
uint64_t pf_topology_num_layers(pf_topology_t t);
uint64_t pf_topology_total_slots(pf_topology_t t);
/* Storage groups (hybrid models), instance.rs:197-220: number of groups, the
 * group of a layer id, and the slots a block of that group needs to seal. */
uint64_t pf_topology_num_groups(pf_topology_t t);
int pf_topology_group_of_layer(pf_topology_t t, uint64_t layer_id, uint32_t* out_group);
int pf_topology_group_total_slots(pf_topology_t t, uint32_t group, uint64_t* out_slots);
int pf_topology_is_page_first(pf_topology_t t);
/* Layer ids are ranks of the byte-wise sorted layer names. */
int pf_topology_layer_id(pf_topology_t t, const char* layer_name, uint64_t* out_id);
int pf_topology_slot_index(pf_topology_t t, uint64_t layer_id, uint64_t tp_rank, uint64_t* out);
int pf_topology_page_placement(pf_topology_t t, uint64_t layer_id, uint64_t* out_offset,
                               uint64_t* out_bytes);
int pf_topology_shard_page_size(pf_topology_t t, uint64_t shard, uint64_t* out);
int pf_topology_shard_layer_count(pf_topology_t t, uint64_t shard, uint64_t* out);

/* ------------------------------------------------------------------------ */
/* Load completion flag in shared memory                                     */
/* Replaces LoadState (pegaflow-core/src/sync_state.rs:23-300): POSIX shm    */
/* object "pega_load_<hex>", magic 'PFLD', version 1, i64 state              */
/* (0 pending, 1 success, -1 error).                                         */
/* ------------------------------------------------------------------------ */

typedef struct pf_load_state_s* pf_load_state_t;

int pf_load_state_create(pf_load_state_t* out);
int pf_load_state_attach(const char* shm_name, pf_load_state_t* out);
int pf_load_state_destroy(pf_load_state_t s);
const char* pf_load_state_name(pf_load_state_t s);
int64_t pf_load_state_get(pf_load_state_t s);
int pf_load_state_set(pf_load_state_t s, int64_t state); /* 1 or -1 */

/* ------------------------------------------------------------------------ */
/* Per-GPU worker pair                                                       */
/* Replaces GpuWorkerPool / LoadTask / SaveTask / LoadCompletion             */
/* (pegaflow-core/src/gpu_worker.rs:15-345,428-523).                         */
/* ------------------------------------------------------------------------ */

typedef struct pf_worker_pool_s* pf_worker_pool_t;
typedef struct pf_task_s* pf_task_t;

/* Ways a task's bytes crossed the link (bits of pf_task_result.paths; a task of
 * mixed layers can carry more than one). */
#define PF_TASK_PATH_STAGED 1u      /* device gather/scatter + DMA copies of a staging slot */
#define PF_TASK_PATH_ZEROCOPY 2u    /* block-ID kernel over mapped host memory */
#define PF_TASK_PATH_DESCRIPTORS 4u /* per-fragment descriptors through a transfer backend */

/* What a settled task reports: the reference's workers log bytes, duration and
 * bandwidth per task (gpu_worker.rs:458-474,505-520); the rest says which way
 * the bytes went and where the task's time was spent, phase by phase. */
typedef struct pf_task_result {
  int32_t status;      /* PF_OK or an error status */
  int32_t done;        /* 0 while pending (only from pf_task_wait with a timeout) */
  uint64_t bytes;      /* payload bytes moved */
  double elapsed_ms;   /* descriptor/plan construction + enqueue + synchronise */
  uint32_t paths;              /* PF_TASK_PATH_* bits */
  uint32_t staged_groups;      /* staging-slot fills: one gather or scatter launch each */
  uint32_t zero_copy_launches; /* launches of the block-ID kernel over host memory */
  uint32_t link_copies;        /* DMA copies of the staged path */
  double resolve_ms;       /* engine loads: leases -> host blocks on the calling thread */
  double queue_ms;         /* submitted -> picked up by the worker thread */
  double convert_ms;       /* worker: host blocks -> block-ID form or descriptors */
  double plan_ms;          /* transfer engine: validation, unit and slab layout */
  double staging_alloc_ms; /* device staging (re)allocated inside the task; 0 once the
                              pool's slots fit (they are allocated when it is spawned) */
  double enqueue_ms;       /* issuing copies and launches (row-order sort included) */
  double sync_ms;          /* last enqueue -> completion event */
  double device_first_ms;  /* on the device: first command of the task -> first staging
                              slot filled (load) or drained (save), or first kernel done */
  double device_ms;        /* on the device: first command -> last command done */
} pf_task_result;

/* GpuWorkerPool::spawn, gpu_worker.rs:131-201: a load thread and a save thread
 * pinned to `numa_node` (< 0 = no pinning), each with its own stream.
 * use_descriptor_backends != 0: per-fragment descriptors through the backend of
 * `transfer_mode`, exactly as the reference (PF_MODE_ZEROCOPY = the kernel
 * backend); 0: the block-ID engine, which picks the way across the link per
 * call (PF_PATH_AUTO) for PF_MODE_DIRECT and PF_MODE_KERNEL alike -- the
 * reference's two modes differ in how they issue the copies, not in the bytes
 * moved, and what they were invented to choose between (one driver call per
 * fragment against one kernel) does not arise here -- and always takes the
 * zero-copy kernel for PF_MODE_ZEROCOPY.
 * Initialisation errors are returned here, synchronously. */
int pf_worker_pool_spawn(int device_id, int numa_node, int transfer_mode,
                         int use_descriptor_backends, pf_worker_pool_t* out);
/* The same with the pool's knobs.  Each worker of a staging pool (block-ID
 * engine, mode direct or kernel) holds two staging slots in device memory,
 * allocated here -- everything a worker needs exists before its first task, as
 * in init_worker (gpu_worker.rs:278-298) -- so a pool costs
 * 2 workers x 2 x staging_slot_bytes of device memory (2 GiB at the default)
 * for as long as it lives, plus 64 MiB each of device and pinned memory for
 * priming the two copy directions. */
typedef struct pf_worker_pool_config {
  int32_t device_id;
  int32_t numa_node;                /* < 0 = no pinning */
  int32_t transfer_mode;            /* PF_MODE_* */
  uint32_t use_descriptor_backends;
  uint64_t staging_slot_bytes;      /* 0 = default (512 MiB); a task's layer larger than a
                                       slot is moved in several fills */
  uint64_t auto_staged_min_bytes;   /* 0 = default (8 MiB), see pf_engine_config */
  uint32_t lazy_staging;            /* 1 = allocate the slots on the first staged task */
  uint32_t side_copy_streams;       /* see pf_engine_config */
} pf_worker_pool_config;
int pf_worker_pool_spawn_ex(const pf_worker_pool_config* cfg, pf_worker_pool_t* out);
/* Device memory the pool's workers hold for staging right now. */
uint64_t pf_worker_pool_staging_bytes(pf_worker_pool_t p);
int pf_worker_pool_destroy(pf_worker_pool_t p);
/* A process's streams share a few hardware queues (GPU_MAX_HW_QUEUES, 4 by
 * default), and kernels of two streams on one queue run one after the other.
 * A pool that is spawned probes its two streams against each other and against
 * the idle worker streams of the pools already on the device, and swaps a
 * stream that clashes for a fresh one, a few times at most.  This is how many
 * clashing pairs were left for this pool (0 = its streams and every stream
 * probed have queues of their own; with more worker streams than hardware
 * queues some pairs must share, and the transfers of those two workers take
 * turns).  No counterpart in the reference, which never checks. */
uint64_t pf_worker_pool_queue_clashes(pf_worker_pool_t p);
/* The same question for all live pools of `device`, asked now: number of worker
 * streams, pairs among the idle ones that share a hardware queue, and streams
 * left out because they were busy.  Probes run on the worker streams
 * themselves: call it while the workers are idle. */
int pf_worker_stream_report(int device, uint64_t* out_streams, uint64_t* out_clashing_pairs,
                            uint64_t* out_skipped);
/* submit_load, gpu_worker.rs:204-212.  The layers are copied; host memory they
 * point to must stay valid until the task settles.  load_state_shm (may be NULL)
 * names a LoadState to signal. */
int pf_worker_submit_load(pf_worker_pool_t p, const pf_layer_transfer* layers, uint64_t n_layers,
                          const char* load_state_shm, pf_task_t* out_task);
/* batch_save, gpu_worker.rs:216-243. */
int pf_worker_submit_save(pf_worker_pool_t p, const pf_layer_transfer* layers, uint64_t n_layers,
                          pf_task_t* out_task);
/* Wait up to timeout_ms (< 0 = forever) for the task to settle.  Returns the
 * task's status once done (message via pf_last_error), PF_OK while pending. */
int pf_task_wait(pf_task_t t, int timeout_ms, pf_task_result* out);
int pf_task_destroy(pf_task_t t);

/* ------------------------------------------------------------------------ */
/* Save / load by block ID                                                   */
/* Replaces the parts of PegaEngine on the path: register_context_layer_     */
/* batch[_strided] (pegaflow-core/src/lib.rs:228-440), batch_save_kv_blocks_ */
/* from_ipc (offload.rs:293-659), prefix query + lease (lib.rs:506-546,      */
/* 614-634), batch_load_kv_blocks_multi_layer[_inproc] (lib.rs:654-898).     */
/* ------------------------------------------------------------------------ */

typedef struct pf_engine_s* pf_engine_t;

typedef struct pf_engine_config {
  uint64_t pool_size;
  uint32_t use_hugepages;
  uint32_t numa_aware;
  uint32_t pool_shards;
  uint32_t blockwise_alloc;          /* one pinned allocation per block */
  uint32_t ssd_enabled;              /* 512-byte host padding + CPU-readable backing */
  uint32_t use_descriptor_backends;  /* see pf_worker_pool_spawn */
  uint64_t unit_size_hint;
  uint64_t lease_ttl_ms;             /* lease.rs:11: 0 = default (600 000 ms) */
  uint64_t auto_staged_min_bytes;    /* workers: a task whose dense layers add up to this much is
                                        staged through device memory instead of moved by the
                                        resident zero-copy kernel (layers of 16 MiB and more are
                                        staged in any case); 0 = default (8 MiB).  Model kernels
                                        that run beside the resident kernel slow down for as long as
                                        it runs, a staged copy leaves them alone: 1 = stage whatever
                                        can be staged, UINT64_MAX = only the large layers. */
  uint64_t staging_slot_bytes;       /* upper bound of a worker's staging slot; 0 = default
                                        (512 MiB).  Every registered context (instance, GPU)
                                        holds 2 workers x 2 slots of min(this, the bytes of all
                                        its registered layers, at least 32 MiB) in device memory
                                        from registration
                                        on -- memory the serving framework's own budget does not
                                        know about. */
  uint32_t lazy_staging;             /* 1 = workers allocate their slots on the first staged
                                        task instead of at registration (that task is slower) */
  uint32_t kernel_mode_zerocopy;     /* 1 = a PF_MODE_KERNEL registration gets zero-copy workers
                                        (PF_MODE_ZEROCOPY), which is what the reference's kernel
                                        mode does (gpu_worker.rs:264-276); 0 = the per-task
                                        choice described at PF_MODE_DIRECT */
  uint32_t side_copy_streams;        /* 0 = default: a worker's link copies run in order on its
                                        one stream, between its gather / scatter kernels.
                                        1 = each worker moves them on a second stream of its
                                        own, so that the copy of one staging fill overlaps the
                                        kernel of the next: a save or a load running alone gains
                                        the kernels' time (Llama-3.1-8B shape: save 55.5 -> 56.2,
                                        load 55.3 -> 56.0 GB/s; a save and a load at once 94.6 ->
                                        88-93 together).  That is four streams per registered
                                        context, and a process's streams share few hardware
                                        queues (GPU_MAX_HW_QUEUES, 4 by default): the pool looks
                                        for queues that no stream of the opposite direction
                                        uses, which gets harder with every further context in
                                        the process, and copy streams of a save and of a load
                                        that do end up on one queue take turns instead of
                                        overlapping.  For processes that hold few contexts per
                                        GPU, or that were started with GPU_MAX_HW_QUEUES=8 (a
                                        save and a load at once then move 96.7-97.4 GB/s, what two
                                        plain hipMemcpyAsync streams do). */
  uint32_t reserved;
} pf_engine_config;

typedef struct pf_layer_save {       /* LayerSave, block.rs:20-25 */
  const char* layer_name;
  const uint64_t* block_ids;
  const uint8_t* const* block_hashes;
  const uint32_t* block_hash_lens;
  uint64_t n_blocks;
} pf_layer_save;

int pf_engine_create(const pf_engine_config* cfg, pf_engine_t* out);
int pf_engine_destroy(pf_engine_t e);
/* block_stride_bytes and layer_group_ids may be NULL. */
int pf_engine_register_context_layer_batch(
    pf_engine_t e, const char* instance_id, const char* namespace_, int device_id,
    uint64_t tp_rank, uint64_t pp_rank, uint64_t tp_size, uint64_t world_size, uint64_t n_layers,
    const char* const* layer_names, const uint64_t* data_ptrs, const uint64_t* size_bytes,
    const uint64_t* num_blocks, const uint64_t* bytes_per_block, const uint64_t* kv_stride_bytes,
    const uint64_t* segments, const uint64_t* block_stride_bytes, const uint32_t* layer_group_ids,
    int transfer_mode, int page_first);
int pf_engine_unregister_instance(pf_engine_t e, const char* instance_id);
/* Returns when the blocks are in host memory and queryable. */
int pf_engine_batch_save(pf_engine_t e, const char* instance_id, uint64_t tp_rank,
                         uint64_t pp_rank, int device_id, const pf_layer_save* saves,
                         uint64_t n_saves);
/* Where the time of the last successful save went; the reference records the
 * same phases as metrics (offload.rs:560-574).  assemble_ms (building the
 * blocks that enter the store) runs while the copy is in flight, inside
 * transfer_ms. */
typedef struct pf_save_profile {
  double validate_ms, filter_ms, alloc_ms, assemble_ms, transfer_ms, publish_ms, total_ms;
  uint64_t bytes;
} pf_save_profile;
int pf_engine_last_save_profile(pf_engine_t e, pf_save_profile* out);
/* The load task that settled last on any worker pool of the engine: bytes,
 * duration (what the reference logs per load, gpu_worker.rs:458-474), the way
 * it crossed the link and its phases.  PF_ERR_STORAGE when no load has settled
 * yet.  The same figures come back from pf_task_wait for the task itself. */
int pf_engine_last_load_profile(pf_engine_t e, pf_task_result* out);
/* Device memory the worker pools of all registered contexts hold for staging. */
uint64_t pf_engine_staging_bytes(pf_engine_t e);
/* Longest cached prefix of the hashes and a lease over those blocks (0 = none). */
int pf_engine_query_prefix(pf_engine_t e, const char* instance_id,
                           const uint8_t* const* hashes, const uint32_t* hash_lens, uint64_t n,
                           uint64_t* out_hits, uint64_t* out_lease);
int pf_engine_release_lease(pf_engine_t e, uint64_t lease);
/* One lease loaded into n_groups load groups.  group_layer_names[g] is an array
 * of group_sizes[g] layer names; dest_block_ids[g] holds one destination per
 * leased block (-1 = skip).  load_state_shm may be NULL.  *out_task settles when
 * the load does. */
int pf_engine_batch_load(pf_engine_t e, const char* instance_id, uint64_t tp_rank, int device_id,
                         uint64_t n_groups, const char* const* const* group_layer_names,
                         const uint64_t* group_sizes, uint64_t lease,
                         const int64_t* const* dest_block_ids, uint64_t n_blocks,
                         const char* load_state_shm, pf_task_t* out_task);
/* The same with several leases in one task (lib.rs:654-898: `loads` is a list
 * of (lease, destinations per group)); dest_block_ids[g] has n_blocks entries,
 * one per block of that lease, -1 = skip. */
typedef struct pf_load_request {
  uint64_t lease;
  const int64_t* const* dest_block_ids;
  uint64_t n_blocks;
} pf_load_request;
int pf_engine_batch_load_multi(pf_engine_t e, const char* instance_id, uint64_t tp_rank,
                               int device_id, uint64_t n_groups,
                               const char* const* const* group_layer_names,
                               const uint64_t* group_sizes, const pf_load_request* loads,
                               uint64_t n_loads, const char* load_state_shm, pf_task_t* out_task);
/* query_group_membership, lib.rs:593-611: out_present[i] = 1 when hashes[i] is
 * sealed in storage group `group` (every position on its own; no prefix rule).
 * An unknown group is an error. */
int pf_engine_query_group_membership(pf_engine_t e, const char* instance_id, uint32_t group,
                                     const uint8_t* const* hashes, const uint32_t* hash_lens,
                                     uint64_t n, uint8_t* out_present);
/* create_query_lease, lib.rs:614-628, naming the blocks by (group, hash): a
 * lease over exactly these blocks, in this order.  n == 0 is an error; a hash
 * that is no longer resident is PF_ERR_STORAGE. */
int pf_engine_create_group_lease(pf_engine_t e, const char* instance_id, uint32_t group,
                                 const uint8_t* const* hashes, const uint32_t* hash_lens,
                                 uint64_t n, uint64_t* out_lease);
/* The two calls above as one step under one lock, which is what the membership
 * branch of the reference's QueryPrefetch handler amounts to (service.rs:606-636
 * leases the very block handles the membership query returned, so no eviction
 * can come between): out_present as pf_engine_query_group_membership, and
 * *out_lease = a lease over exactly the present blocks in list order, or 0 when
 * none is present, or when require_all != 0 and one is missing. */
int pf_engine_query_group_lease(pf_engine_t e, const char* instance_id, uint32_t group,
                                const uint8_t* const* hashes, const uint32_t* hash_lens,
                                uint64_t n, int require_all, uint8_t* out_present,
                                uint64_t* out_lease);
int pf_engine_pool_usage(pf_engine_t e, uint64_t* out_used, uint64_t* out_total);
uint64_t pf_engine_cached_blocks(pf_engine_t e);
/* Blocks that hold some but not all of their slots (saves of the remaining
 * layers or ranks are still expected). */
uint64_t pf_engine_inflight_blocks(pf_engine_t e);
/* gc_stale_inflight, storage/write_path.rs:52-61,302-330: drop the incomplete
 * blocks whose first slot arrived more than max_age_ms ago, returning their
 * pinned memory; returns how many.  The reference's server calls this
 * periodically. */
uint64_t pf_engine_gc_stale_inflight(pf_engine_t e, uint64_t max_age_ms);
/* Drop every cached block that is not leased; returns how many. */
uint64_t pf_engine_evict_all(pf_engine_t e);
/* Query leases expire (lease.rs:11-12,47,91-118,174-181): a lease that is not
 * consumed within lease_ttl_ms stops protecting its blocks from eviction, and
 * a load that names it afterwards fails with "query lease is unknown or
 * expired".  Expired leases are dropped whenever a lease is created, consumed
 * or released, before a save gives up for lack of pinned memory, by
 * pf_engine_gc_stale_inflight, and by this call, which stands in for the
 * reference's 30-second sweeper task; returns how many were dropped. */
uint64_t pf_engine_sweep_expired_leases(pf_engine_t e);
/* Leases that have not been consumed, released or swept. */
uint64_t pf_engine_live_leases(pf_engine_t e);

/* ------------------------------------------------------------------------ */
/* Device memory handed over by another process                              */
/* Replaces CudaIPCWrapper (python/pegaflow/ipc_wrapper.py:102-160) and      */
/* CudaTensorRegistry (pegaflow-server/src/registry.rs:45-203): the worker   */
/* process exports the allocation behind each KV cache tensor, the server    */
/* process opens it and registers the mapped address with the engine         */
/* (pegaflow-server/src/service.rs:205-336, RegisterContextBatch).           */
/* ------------------------------------------------------------------------ */

/* What a worker sends per layer in place of the reference's pickled wrapper:
 * IPC handle of the allocation, where the tensor's storage sits in it, and the
 * UUID of the GPU (device ordinals differ between processes). */
typedef struct pf_ipc_tensor {
  uint8_t handle[64];      /* hipIpcMemHandle_t */
  uint64_t alloc_size;     /* bytes of the exported allocation */
  uint64_t offset;         /* storage start inside the allocation */
  uint64_t size_bytes;     /* storage bytes (the engine's size_bytes) */
  uint8_t device_uuid[16];
} pf_ipc_tensor;

int pf_device_uuid(int device, uint8_t out_uuid[16]);
/* ipc_wrapper.py:75-98: ordinal of the device with this UUID in this process. */
int pf_device_from_uuid(const uint8_t uuid[16], int* out_device);
/* Worker side (CudaIPCWrapper.__init__): describe [dev_ptr, +size_bytes), which
 * lies inside one device allocation of this process.  Keep an allocation that
 * is shared this way below 2 GiB. */
int pf_ipc_export(uint64_t dev_ptr, uint64_t size_bytes, pf_ipc_tensor* out);

typedef struct pf_tensor_registry_s* pf_tensor_registry_t;

int pf_registry_create(pf_tensor_registry_t* out);
/* Closes every mapping it still holds. */
int pf_registry_destroy(pf_tensor_registry_t r);
/* register_layers, registry.rs:67-107: open each layer's allocation (once per
 * allocation) on device_id and return the mapped data_ptr / size_bytes per
 * layer.  Errors with the reference's wording: "context {key} is already
 * registered", "layer {name} appears more than once in context {key}",
 * "context {key} is pinned to device {a} but got {b}".  On error nothing stays
 * mapped. */
int pf_registry_register_layers(pf_tensor_registry_t r, const char* context_key, int device_id,
                                uint64_t n_layers, const char* const* layer_names,
                                const pf_ipc_tensor* tensors, uint64_t* out_data_ptrs,
                                uint64_t* out_size_bytes);
/* registry.rs:108-171; each returns the number of tensors released.  An
 * instance's contexts are the keys that start with "{instance_id}:". */
uint64_t pf_registry_drop_context(pf_tensor_registry_t r, const char* context_key);
uint64_t pf_registry_drop_instance(pf_tensor_registry_t r, const char* instance_id);
uint64_t pf_registry_clear(pf_tensor_registry_t r);
uint64_t pf_registry_context_count(pf_tensor_registry_t r);
/* The RegisterContextBatch handler (service.rs:205-336): validate, open the
 * tensors under the context key "{instance}:tp{r}:pp{p}:dev{d}", register the
 * mapped addresses with the engine, and roll the mappings back when the engine
 * refuses.  layer_group_ids may be NULL. */
int pf_server_register_context_batch(
    pf_engine_t e, pf_tensor_registry_t r, const char* instance_id, const char* namespace_,
    int device_id, uint64_t tp_rank, uint64_t pp_rank, uint64_t tp_size, uint64_t world_size,
    uint64_t n_layers, const char* const* layer_names, const pf_ipc_tensor* tensors,
    const uint64_t* num_blocks, const uint64_t* bytes_per_block, const uint64_t* kv_stride_bytes,
    const uint64_t* segments, const uint32_t* layer_group_ids, int transfer_mode, int page_first);

#ifdef __cplusplus
} /* extern "C" */
#endif
#endif /* PEGAHIP_H */
