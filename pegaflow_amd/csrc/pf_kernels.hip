// gfx950 copy kernels of the KV block transfer path.
//
// All of them are pure byte movers bounded by HBM (device <-> device staging)
// or by the host link (device <-> mapped pinned host memory).  Shape:
//   * a workgroup is 256 lanes = 4 wavefronts of 64;
//   * a tile is 256 lanes x U x 16 bytes; every lane issues its U 16-byte
//     loads before the first store so U global_load_dwordx4 are in flight per
//     lane, and consecutive lanes touch consecutive 16-byte words, so each
//     wavefront's access is one 1 KiB contiguous burst;
//   * loads are non-temporal and stores "sc1 nt": the data is touched once;
//   * all per-tile address arithmetic is wave-uniform (scalar registers).
#include "pf_kernels.hpp"

#include <mutex>

#include "pf_common.hpp"

namespace pf {

namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
// Address-space-1 (global) views, so the compiler emits global_load/store
// instead of flat accesses for addresses that arrive as integers.
typedef __attribute__((address_space(1))) u32x4 g_u32x4;
typedef __attribute__((address_space(1))) unsigned int g_u32;
typedef __attribute__((address_space(1))) unsigned char g_u8;
// Address-space-4 (constant) views for the read-only, wave-uniform id list
// and page table: uniform constant loads become scalar loads.
typedef __attribute__((address_space(4))) const uint32_t c_u32;
typedef __attribute__((address_space(4))) const uint64_t c_u64;
typedef __attribute__((address_space(4))) const BlockUnit c_unit;

constexpr int kLanes = 256;
constexpr uint32_t kMaxRowUnits = kRowsLaunchUnits;  // units of one block_tiles_rows_kernel launch

// 16-byte store with the cache policy "sc1 nt".  Measured on MI355X at the
// Llama shape (5000 x 2 x 32 KiB gathered or scattered per launch) over all 49
// load x store policy pairs: a destination written in ascending address order
// is written fastest with "sc1 nt" (gather 6.35 TB/s against 6.30 for plain
// nt; scatter in ascending-id row order 6.17 against 5.63 for "sc1" and 5.44
// for an ordinary store).  Stores into mapped host memory want the same: every
// policy with sc1 moves the Llama layer over the link at 56.3 GB/s (64
// workgroups; hipMemcpyAsync on the same box 56.1), plain and sc0 stores at
// 54.2, nt alone at 53.9; loads from host memory do not care (56.6 with any
// policy).
//
// The policy bits are not reachable from a plain C++ store, and the store must
// not be inline assembly: the compiler cannot see that an asm statement is a
// 16-byte store, so it neither keeps the data registers alive for the wait
// states such a store needs nor counts it for s_waitcnt.  (With the store
// written as asm, a four-store tile loop had the address of the fourth store
// computed into the data registers of the first two instructions after that
// one was issued, and the first store wrote address bits into lanes 12-15 of
// every 16-lane row.)  A raw buffer store carries the bits in its `aux`
// operand and is an ordinary instruction to the compiler.  The descriptor
// covers exactly the tile (wave-uniform base and byte count, no stride), so a
// store beyond the tile would be dropped by the hardware's range check.
constexpr int kAuxSc1Nt = (1 << 4) | (1 << 1);  // gfx940+: bit 4 = sc1, bit 1 = nt
constexpr int kRawBufferWord3 = 0x00020000;     // untyped 32-bit data, no swizzle, no tid

__device__ __forceinline__ __amdgpu_buffer_rsrc_t tile_descriptor(uint64_t base, uint32_t bytes) {
  // The base is wave-uniform by construction; say so, or the compiler would
  // loop over the lanes to build one descriptor per distinct value.
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(base));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(base >> 32));
  return __builtin_amdgcn_make_buffer_rsrc(
      reinterpret_cast<void*>((static_cast<uint64_t>(hi) << 32) | lo), 0,
      static_cast<int>(__builtin_amdgcn_readfirstlane(bytes)), kRawBufferWord3);
}

__device__ __forceinline__ void store16_sc1_nt(__amdgpu_buffer_rsrc_t tile, uint32_t offset,
                                               u32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(v, tile, static_cast<int>(offset), 0, kAuxSc1Nt);
}

// Copy `bytes` <= U*4096 from src to dst; both 16-byte aligned.
template <int U>
__device__ __forceinline__ void copy_tile_vec(uint64_t dst, uint64_t src, uint32_t bytes) {
  constexpr uint32_t kTile = U * kLanes * 16;
  const uint32_t lane = threadIdx.x;
  const g_u32x4* __restrict__ s = reinterpret_cast<const g_u32x4*>(src);
  u32x4 v[U];
  const __amdgpu_buffer_rsrc_t tile = tile_descriptor(dst, bytes & ~15u);
  if (bytes == kTile) {
#pragma unroll
    for (int k = 0; k < U; ++k) v[k] = __builtin_nontemporal_load(s + lane + k * kLanes);
#pragma unroll
    for (int k = 0; k < U; ++k) store16_sc1_nt(tile, (lane + k * kLanes) * 16u, v[k]);
    return;
  }
  const uint32_t nvec = bytes >> 4;
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t idx = lane + k * kLanes;
    if (idx < nvec) v[k] = __builtin_nontemporal_load(s + idx);
  }
#pragma unroll
  for (int k = 0; k < U; ++k) {
    const uint32_t idx = lane + k * kLanes;
    if (idx < nvec) store16_sc1_nt(tile, idx * 16u, v[k]);
  }
  // Fewer than 16 trailing bytes (fragment size not a multiple of 16).
  const uint32_t j = (nvec << 4) + lane;
  if (j < bytes) {
    reinterpret_cast<g_u8*>(dst)[j] = reinterpret_cast<const g_u8*>(src)[j];
  }
}

// Copy `bytes` with no alignment assumption: 4-byte words when both sides
// allow it, single bytes otherwise.
__device__ __forceinline__ void copy_tile_any(uint64_t dst, uint64_t src, uint32_t bytes) {
  const uint32_t lane = threadIdx.x;
  const g_u8* __restrict__ sb = reinterpret_cast<const g_u8*>(src);
  g_u8* __restrict__ db = reinterpret_cast<g_u8*>(dst);
  if (((dst | src) & 3ull) == 0) {
    const uint32_t nword = bytes >> 2;
    const g_u32* __restrict__ s = reinterpret_cast<const g_u32*>(src);
    g_u32* __restrict__ d = reinterpret_cast<g_u32*>(dst);
    for (uint32_t j = lane; j < nword; j += kLanes) d[j] = s[j];
    for (uint32_t j = (nword << 2) + lane; j < bytes; j += kLanes) db[j] = sb[j];
  } else {
    for (uint32_t j = lane; j < bytes; j += kLanes) db[j] = sb[j];
  }
}

// Descriptor-table copy: table[3i..3i+2] = dst, src, size.  blockIdx.x strides
// over descriptors, blockIdx.y over the tiles inside one descriptor, so a
// batch of few large copies still spreads over the whole chip.  The row a
// workgroup handles next is fetched before the current one is copied: the
// table may sit in mapped host memory (short batches skip the upload), where
// a row is a couple of microseconds away.
template <int U>
__global__ __launch_bounds__(kLanes) void desc_copy_kernel(const uint64_t* __restrict__ table,
                                                           uint32_t n) {
  constexpr uint64_t kTile = static_cast<uint64_t>(U) * kLanes * 16;
  uint32_t i = blockIdx.x;
  if (i >= n) return;
  uint64_t dst = table[3ull * i + 0];
  uint64_t src = table[3ull * i + 1];
  uint64_t size = table[3ull * i + 2];
  for (;;) {
    const uint32_t next = i + gridDim.x;
    uint64_t next_dst = 0, next_src = 0, next_size = 0;
    if (next < n) {
      next_dst = table[3ull * next + 0];
      next_src = table[3ull * next + 1];
      next_size = table[3ull * next + 2];
    }
    const uint64_t n_tiles = (size + kTile - 1) / kTile;
    const bool vec = ((dst | src) & 15ull) == 0;
    for (uint64_t t = blockIdx.y; t < n_tiles; t += gridDim.y) {
      const uint64_t off = t * kTile;
      const uint64_t left = size - off;
      const uint32_t bytes = left < kTile ? static_cast<uint32_t>(left) : static_cast<uint32_t>(kTile);
      if (vec) {
        copy_tile_vec<U>(dst + off, src + off, bytes);
      } else {
        copy_tile_any(dst + off, src + off, bytes);
      }
    }
    if (next >= n) break;
    i = next;
    dst = next_dst;
    src = next_src;
    size = next_size;
  }
}

// The same copy over caller-format descriptors (pf_copy_desc, 48 bytes each):
// the table is the caller's array as it is, so the host side repacks nothing.
// HOST_IS_SRC picks which of the two device-visible addresses is the source.
template <int U, bool HOST_IS_SRC>
__global__ __launch_bounds__(kLanes) void desc48_copy_kernel(
    const pf_copy_desc* __restrict__ table, uint32_t n) {
  constexpr uint64_t kTile = static_cast<uint64_t>(U) * kLanes * 16;
  uint32_t i = blockIdx.x;
  if (i >= n) return;
  uint64_t near_addr = table[i].device;
  uint64_t far_addr = table[i].host_device;
  uint64_t size = table[i].size;
  for (;;) {
    // The next row is on its way while this one is copied.
    const uint32_t next = i + gridDim.x;
    uint64_t next_near = 0, next_far = 0, next_size = 0;
    if (next < n) {
      next_near = table[next].device;
      next_far = table[next].host_device;
      next_size = table[next].size;
    }
    const uint64_t dst = HOST_IS_SRC ? near_addr : far_addr;
    const uint64_t src = HOST_IS_SRC ? far_addr : near_addr;
    const uint64_t n_tiles = (size + kTile - 1) / kTile;
    const bool vec = ((dst | src) & 15ull) == 0;
    for (uint64_t t = blockIdx.y; t < n_tiles; t += gridDim.y) {
      const uint64_t off = t * kTile;
      const uint64_t left = size - off;
      const uint32_t bytes = left < kTile ? static_cast<uint32_t>(left) : static_cast<uint32_t>(kTile);
      if (vec) {
        copy_tile_vec<U>(dst + off, src + off, bytes);
      } else {
        copy_tile_any(dst + off, src + off, bytes);
      }
    }
    if (next >= n) break;
    i = next;
    near_addr = next_near;
    far_addr = next_far;
    size = next_size;
  }
}

// Block-ID gather / scatter over mapped host memory (the zero-copy form).  The
// grid is a few rows of workgroups, as many workgroups in all as the launch
// may keep on the device.  Row y walks the units y, y + rows, ... one after the
// other and its workgroups stride over the tiles of each, so the workgroup
// count does not grow with the number of units.  With large units there is one
// row and the units complete in order; a call of many small units (a few
// blocks of every layer, the shape of a decode-time load) gets several rows,
// or most workgroups would find no tile in a unit of four tiles and the rest
// would walk all the units alone: 32 layers x 1 block loaded in 68 us with one
// row of 16 workgroups (4 of them busy, 32 tiles each one after the other,
// every tile a round trip over the link).  Tile order inside a unit is
// (segment, list position, tile in fragment), so at any moment the workgroups
// of a row touch neighbouring far-side addresses.
template <int U, bool TO_FAR, typename UnitPtr>
__device__ __forceinline__ void block_units_body(UnitPtr units, uint32_t n_units, uint64_t bias) {
  constexpr uint64_t kTile = static_cast<uint64_t>(U) * kLanes * 16;
  for (uint32_t unit = blockIdx.y; unit < n_units; unit += gridDim.y) {
    // Every field below is wave-uniform: read once into scalar registers.
    UnitPtr up = units + unit;
    const uint64_t near_base = up->near_base;
    const uint64_t block_stride = up->block_stride;
    const uint64_t kv_stride = up->kv_stride;
    const uint64_t frag_bytes = up->frag_bytes;
    const uint64_t far_base0 = up->far_base[0];
    const uint64_t far_base1 = up->far_base[1];
    const uint64_t far_stride = up->far_stride;
    c_u32* ids = reinterpret_cast<c_u32*>(reinterpret_cast<uint64_t>(up->ids) + bias);
    const bool paged = up->far_table != nullptr;
    c_u64* far_table =
        reinterpret_cast<c_u64*>(reinterpret_cast<uint64_t>(up->far_table) + (paged ? bias : 0));
    const uint64_t far_table_off = up->far_table_off;
    const uint32_t tiles_per_frag = up->tiles_per_frag;
    const bool vec_ok = up->vec_ok != 0;
    const bool ids16 = up->ids16 != 0;
    // The host keeps a unit's tile count below 2^32, so 32-bit scalar division.
    const uint32_t tiles_per_seg = up->n_blocks * tiles_per_frag;
    const uint32_t n_tiles = tiles_per_seg * up->n_seg;
    for (uint32_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
      const uint32_t seg = t >= tiles_per_seg ? 1u : 0u;
      const uint32_t r = seg ? t - tiles_per_seg : t;
      // The quotient is wave-uniform; pin it to a scalar register so the id and
      // page-table reads below are scalar loads.
      const uint32_t pos = __builtin_amdgcn_readfirstlane(r / tiles_per_frag);
      const uint32_t c = r - pos * tiles_per_frag;
      const uint64_t off = static_cast<uint64_t>(c) * kTile;
      const uint64_t left = frag_bytes - off;
      const uint32_t bytes = left < kTile ? static_cast<uint32_t>(left) : static_cast<uint32_t>(kTile);
      // 16-bit ids sit two to a word (there is no scalar load of half a word).
      const uint32_t id_word = ids[ids16 ? pos >> 1 : pos];
      const uint64_t id = ids16 ? ((pos & 1u) ? id_word >> 16 : id_word & 0xFFFFu) : id_word;
      const uint64_t near_addr = near_base + id * block_stride + (seg ? kv_stride : 0) + off;
      uint64_t far_addr;
      if (paged) {
        far_addr = far_table[pos] + far_table_off + (seg ? frag_bytes : 0) + off;
      } else {
        far_addr = (seg ? far_base1 : far_base0) + static_cast<uint64_t>(pos) * far_stride + off;
      }
      const uint64_t dst = TO_FAR ? far_addr : near_addr;
      const uint64_t src = TO_FAR ? near_addr : far_addr;
      if (vec_ok) {
        copy_tile_vec<U>(dst, src, bytes);
      } else {
        copy_tile_any(dst, src, bytes);
      }
    }
  }
}

template <int U, bool TO_FAR>
__global__ __launch_bounds__(kLanes) void block_units_kernel(const BlockUnit* __restrict__ units,
                                                             uint32_t n_units) {
  block_units_body<U, TO_FAR, const BlockUnit*>(units, n_units, 0);
}

// The same kernel for short lists, with the units, id lists and page tables
// travelling in the kernel's arguments instead of a slab that has to be
// uploaded first: one command fewer on the stream (measured on MI355X, submit +
// synchronise of one small transfer: the upload costs 3.5 us of ~36 us at 1 MiB
// and of ~90 us at 4 MiB).  `slab` is the first argument, so it starts at
// offset 0 of the argument segment; a unit's `ids` / `far_table` hold byte
// offsets into it.
template <int U, bool TO_FAR>
__global__ __launch_bounds__(kLanes) void block_units_args_kernel(ArgSlab slab, uint32_t first_unit,
                                                                  uint32_t n_units) {
  (void)slab;
  const uint64_t base = reinterpret_cast<uint64_t>(__builtin_amdgcn_kernarg_segment_ptr());
  block_units_body<U, TO_FAR, c_unit*>(reinterpret_cast<c_unit*>(base) + first_unit, n_units, base);
}

// Block-ID gather / scatter, one small tile per workgroup (the HBM-bound form
// used between the KV cache and a device staging buffer).
//
// grid = (tiles per fragment, list positions, SEGS * units), SEGS being the
// largest segment count among the units of the launch; a workgroup of LT
// lanes moves LT*16 bytes with one 16-byte load per lane.  Measured on MI355X
// against the alternatives at the Llama shape (5000 x 2 x 32 KiB per launch):
// this form reaches ~6.3 TB/s (read+write), a 16 KiB-per-workgroup grid-stride
// loop ~5.6 TB/s, a persistent grid ~5.5 TB/s; the tiny register footprint
// keeps every SIMD full of waves, and the 3-D grid needs no division.
// Remapping workgroups so that each XCD owns whole fragments changed nothing
// (no data is reused, so there is no L2 locality to win).
// UNITS_INNER: grid.y walks the (unit, segment) pairs and grid.z the list
// positions, so workgroups that are dispatched together belong to one
// position; otherwise grid.y walks the positions of one (unit, segment).
// One tile of one fragment: row `row` of unit `up`, segment `seg`, tile blockIdx.x.
template <int LT, bool TO_FAR, typename UnitPtr>
__device__ __forceinline__ void block_tiles_copy(UnitPtr up, uint32_t row, uint32_t seg) {
  constexpr uint32_t kTile = LT * 16;
  if (row >= up->n_blocks) return;
  // Rows may visit the list positions in another order (see launch_block_tiles).
  uint32_t pos = row;
  if (up->order != nullptr) {
    c_u32* order = reinterpret_cast<c_u32*>(reinterpret_cast<uint64_t>(up->order));
    pos = order[row];
  }
  const uint64_t frag_bytes = up->frag_bytes;
  const uint64_t off = static_cast<uint64_t>(blockIdx.x) * kTile;
  if (seg >= up->n_seg || pos >= up->n_blocks || off >= frag_bytes) return;
  c_u32* ids = reinterpret_cast<c_u32*>(reinterpret_cast<uint64_t>(up->ids));
  const uint64_t id = ids[pos];
  const uint64_t near_addr =
      up->near_base + id * up->block_stride + (seg ? up->kv_stride : 0) + off;
  uint64_t far_addr;
  if (up->far_table != nullptr) {
    c_u64* far_table = reinterpret_cast<c_u64*>(reinterpret_cast<uint64_t>(up->far_table));
    far_addr = far_table[pos] + up->far_table_off + (seg ? frag_bytes : 0) + off;
  } else {
    far_addr = (seg ? up->far_base[1] : up->far_base[0]) +
               static_cast<uint64_t>(pos) * up->far_stride + off;
  }
  const uint64_t dst = TO_FAR ? far_addr : near_addr;
  const uint64_t src = TO_FAR ? near_addr : far_addr;
  const uint64_t left = frag_bytes - off;
  const uint32_t bytes = left < kTile ? static_cast<uint32_t>(left) : kTile;
  const uint32_t lane = threadIdx.x;
  if (up->vec_ok) {
    const g_u32x4* __restrict__ s = reinterpret_cast<const g_u32x4*>(src);
    const uint32_t nvec = bytes >> 4;
    const __amdgpu_buffer_rsrc_t tile = tile_descriptor(dst, nvec << 4);
    if (lane < nvec) {
      // Streaming load and store in both directions: nothing is read twice.
      // (Gather with an ordinary load of the scattered source: 5.90 TB/s at
      // the Llama shape, with the streaming load 6.14.)
      const u32x4 v = __builtin_nontemporal_load(s + lane);
      store16_sc1_nt(tile, lane * 16u, v);
    }
    const uint32_t j = (nvec << 4) + lane;
    if (j < bytes) reinterpret_cast<g_u8*>(dst)[j] = reinterpret_cast<const g_u8*>(src)[j];
  } else {
    const g_u8* __restrict__ sb = reinterpret_cast<const g_u8*>(src);
    g_u8* __restrict__ db = reinterpret_cast<g_u8*>(dst);
    if (((dst | src) & 3ull) == 0) {
      const uint32_t nword = bytes >> 2;
      const g_u32* __restrict__ sw = reinterpret_cast<const g_u32*>(src);
      g_u32* __restrict__ dw = reinterpret_cast<g_u32*>(dst);
      for (uint32_t j = lane; j < nword; j += LT) dw[j] = sw[j];
      for (uint32_t j = (nword << 2) + lane; j < bytes; j += LT) db[j] = sb[j];
    } else {
      for (uint32_t j = lane; j < bytes; j += LT) db[j] = sb[j];
    }
  }
}

template <int LT, bool TO_FAR, int SEGS, bool UNITS_INNER, typename UnitPtr>
__device__ __forceinline__ void block_tiles_body(UnitPtr units) {
  const uint32_t unit_seg = UNITS_INNER ? blockIdx.y : blockIdx.z;
  const uint32_t row = UNITS_INNER ? blockIdx.z : blockIdx.y;
  UnitPtr up = units + (SEGS == 2 ? unit_seg >> 1 : unit_seg);
  const uint32_t seg = SEGS == 2 ? (unit_seg & 1u) : 0u;
  block_tiles_copy<LT, TO_FAR, UnitPtr>(up, row, seg);
}

template <int LT, bool TO_FAR, int SEGS, bool UNITS_INNER>
__global__ __launch_bounds__(LT) void block_tiles_kernel(const BlockUnit* __restrict__ units) {
  block_tiles_body<LT, TO_FAR, SEGS, UNITS_INNER, const BlockUnit*>(units);
}

// A few units of different lengths in one launch (the fills of a staging slot:
// the tail of one layer, whole layers, the head of the next): grid.y runs over
// the rows of all units laid end to end, so that no workgroup is launched for a
// row a shorter unit does not have (with the grid of block_tiles_kernel, sized
// by the longest unit, up to 45 % of the workgroups of such a launch found
// nothing to do and it ran at 5.2 instead of 6.1 TB/s).  The running row counts
// arrive with the kernel's arguments, so finding the unit costs no memory access.
struct RowEnds {
  uint32_t end[kMaxRowUnits];  // end[k] = rows of units 0..k; UINT32_MAX past the last unit
};

template <int LT, bool TO_FAR, int SEGS>
__global__ __launch_bounds__(LT) void block_tiles_rows_kernel(const BlockUnit* __restrict__ units,
                                                              RowEnds ends) {
  // More rows than one grid extent are folded over grid.z: z = chunk * SEGS + segment.
  const uint32_t chunk = SEGS == 2 ? blockIdx.z >> 1 : blockIdx.z;
  const uint32_t seg = SEGS == 2 ? blockIdx.z & 1u : 0u;
  const uint32_t row = chunk * gridDim.y + blockIdx.y;
  uint32_t unit = 0, first = 0;
#pragma unroll
  for (uint32_t k = 0; k + 1 < kMaxRowUnits; ++k) {
    if (row >= ends.end[k]) {
      unit = k + 1;
      first = ends.end[k];
    }
  }
  // (A row past the last unit's end, in the last chunk, finds no block there.)
  block_tiles_copy<LT, TO_FAR, const BlockUnit*>(units + unit, row - first, seg);
}

// One unit, passed by value: its fields arrive with the kernel's arguments
// instead of behind a pointer, one dependent scalar load fewer before the id of
// the workgroup's row is known (a workgroup lives for one load and one store, so
// every level of that chain is a measurable part of its life).  The unit is the
// first argument: offset 0 of the argument segment.
template <int LT, bool TO_FAR, int SEGS>
__global__ __launch_bounds__(LT) void block_tiles_one_kernel(BlockUnit unit) {
  (void)unit;
  block_tiles_body<LT, TO_FAR, SEGS, false, c_unit*>(
      reinterpret_cast<c_unit*>(reinterpret_cast<uint64_t>(__builtin_amdgcn_kernarg_segment_ptr())));
}

// The two halves of streams_run_concurrently().  The wait is bounded by the
// constant-rate device clock (100 MHz), so the lane leaves whatever happens.
__global__ __launch_bounds__(64) void probe_wait_kernel(uint32_t* word, uint32_t* seen,
                                                        uint64_t max_ticks) {
  if (threadIdx.x != 0) return;
  const uint64_t begin = wall_clock64();
  uint32_t value = 0;
  for (;;) {
    value = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (value != 0 || wall_clock64() - begin > max_ticks) break;
    __builtin_amdgcn_s_sleep(16);
  }
  __hip_atomic_store(seen, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

__global__ __launch_bounds__(64) void probe_post_kernel(uint32_t* word) {
  if (threadIdx.x == 0) __hip_atomic_store(word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int U>
__global__ __launch_bounds__(kLanes) void plain_copy_kernel(uint64_t dst, uint64_t src,
                                                            uint64_t bytes) {
  constexpr uint64_t kTile = static_cast<uint64_t>(U) * kLanes * 16;
  const uint64_t n_tiles = (bytes + kTile - 1) / kTile;
  for (uint64_t t = blockIdx.x; t < n_tiles; t += gridDim.x) {
    const uint64_t off = t * kTile;
    const uint64_t left = bytes - off;
    copy_tile_vec<U>(dst + off, src + off,
                     left < kTile ? static_cast<uint32_t>(left) : static_cast<uint32_t>(kTile));
  }
}

// Plain copy in the one-tile-per-workgroup form of block_tiles_kernel.
template <int LT>
__global__ __launch_bounds__(LT) void plain_tiles_kernel(uint64_t dst, uint64_t src,
                                                         uint64_t bytes) {
  const uint64_t off = static_cast<uint64_t>(blockIdx.x) * (LT * 16ull) + threadIdx.x * 16ull;
  if (off < bytes) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const g_u32x4*>(src + off));
    __builtin_nontemporal_store(v, reinterpret_cast<g_u32x4*>(dst + off));
  }
}

constexpr int kTileLanes = 128;  // lanes of a block_tiles_kernel workgroup
static_assert(kTileLanes * 16 == kStagedTileBytes, "tile size the planner of launches assumes");
constexpr uint32_t kMaxGridX = 1u << 22;  // the kernels grid-stride past this
constexpr int kDescUnroll = 4;

}  // namespace

bool unroll_supported(int unroll) { return unroll == 1 || unroll == 2 || unroll == 4 || unroll == 8; }

namespace {
// Grid of a zero-copy launch: `max_workgroups` (0 = no cap) in all; x strides
// over the tiles of a unit, y over the units.  Units as large as the cap or
// larger leave one row.
dim3 block_units_grid(uint32_t n_units, uint64_t max_tiles, uint32_t max_workgroups) {
  uint64_t gx = max_tiles < kMaxGridX ? max_tiles : kMaxGridX;
  if (max_workgroups != 0 && gx > max_workgroups) gx = max_workgroups;
  uint64_t gy = 1;
  if (max_workgroups != 0 && gx < max_workgroups) {
    gy = max_workgroups / gx;
    if (gy > n_units) gy = n_units;
    if (gy > 65535) gy = 65535;
    if (gy < 1) gy = 1;
  }
  return dim3(static_cast<uint32_t>(gx), static_cast<uint32_t>(gy), 1);
}
}  // namespace

int launch_desc_copy(const uint64_t* table, uint64_t n, uint64_t max_size, hipStream_t s,
                     uint32_t max_workgroups);

int launch_block_units(const BlockUnit* units, uint32_t n_units, uint64_t max_tiles, bool to_far,
                       int unroll, uint32_t max_workgroups_x, hipStream_t s) {
  if (n_units == 0 || max_tiles == 0) return PF_OK;
  if (max_tiles > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "unit of %llu tiles exceeds the kernel limit",
                static_cast<unsigned long long>(max_tiles));
  }
  const dim3 grid = block_units_grid(n_units, max_tiles, max_workgroups_x);
  dim3 block(kLanes, 1, 1);
#define PF_LAUNCH_UNITS(U_)                                                                   \
  case U_:                                                                                    \
    if (to_far) {                                                                             \
      hipLaunchKernelGGL((block_units_kernel<U_, true>), grid, block, 0, s, units, n_units);  \
    } else {                                                                                  \
      hipLaunchKernelGGL((block_units_kernel<U_, false>), grid, block, 0, s, units, n_units); \
    }                                                                                         \
    break;
  switch (unroll) {
    PF_LAUNCH_UNITS(1)
    PF_LAUNCH_UNITS(2)
    PF_LAUNCH_UNITS(4)
    PF_LAUNCH_UNITS(8)
    default:
      return fail(PF_ERR_INVALID_ARGUMENT, "unsupported tile unroll %d", unroll);
  }
#undef PF_LAUNCH_UNITS
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "block_units_kernel launch");
  return PF_OK;
}

int launch_block_units_args(const ArgSlab& slab, uint32_t first_unit, uint32_t n_units,
                            uint64_t max_tiles, bool to_far, int unroll, uint32_t max_workgroups_x,
                            hipStream_t s) {
  if (n_units == 0 || max_tiles == 0) return PF_OK;
  if (max_tiles > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "unit of %llu tiles exceeds the kernel limit",
                static_cast<unsigned long long>(max_tiles));
  }
  const dim3 grid = block_units_grid(n_units, max_tiles, max_workgroups_x);
  dim3 block(kLanes, 1, 1);
#define PF_LAUNCH_ARGS(U_)                                                                       \
  case U_:                                                                                       \
    if (to_far) {                                                                                \
      hipLaunchKernelGGL((block_units_args_kernel<U_, true>), grid, block, 0, s, slab,           \
                         first_unit, n_units);                                                   \
    } else {                                                                                     \
      hipLaunchKernelGGL((block_units_args_kernel<U_, false>), grid, block, 0, s, slab,          \
                         first_unit, n_units);                                                   \
    }                                                                                            \
    break;
  switch (unroll) {
    PF_LAUNCH_ARGS(1)
    PF_LAUNCH_ARGS(2)
    PF_LAUNCH_ARGS(4)
    PF_LAUNCH_ARGS(8)
    default:
      return fail(PF_ERR_INVALID_ARGUMENT, "unsupported tile unroll %d", unroll);
  }
#undef PF_LAUNCH_ARGS
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "block_units_args_kernel launch");
  return PF_OK;
}

int launch_block_tiles_one(const BlockUnit& unit, bool to_far, hipStream_t s) {
  if (unit.n_blocks == 0 || unit.frag_bytes == 0) return PF_OK;
  if (unit.n_seg != 1 && unit.n_seg != 2) {
    return fail(PF_ERR_INVALID_ARGUMENT, "tile launch: %u segments per block", unit.n_seg);
  }
  constexpr uint64_t kTile = kTileLanes * 16;
  const uint64_t gx = (unit.frag_bytes + kTile - 1) / kTile;
  if (unit.n_blocks > kMaxTileBlocks || gx > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT, "tile launch out of range: %u blocks, %llu-byte fragments",
                unit.n_blocks, static_cast<unsigned long long>(unit.frag_bytes));
  }
  dim3 grid(static_cast<uint32_t>(gx), unit.n_blocks, unit.n_seg);
  dim3 block(kTileLanes, 1, 1);
  if (unit.n_seg == 2) {
    if (to_far) {
      hipLaunchKernelGGL((block_tiles_one_kernel<kTileLanes, true, 2>), grid, block, 0, s, unit);
    } else {
      hipLaunchKernelGGL((block_tiles_one_kernel<kTileLanes, false, 2>), grid, block, 0, s, unit);
    }
  } else if (to_far) {
    hipLaunchKernelGGL((block_tiles_one_kernel<kTileLanes, true, 1>), grid, block, 0, s, unit);
  } else {
    hipLaunchKernelGGL((block_tiles_one_kernel<kTileLanes, false, 1>), grid, block, 0, s, unit);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "block_tiles_one_kernel launch");
  return PF_OK;
}

int launch_block_tiles_rows(const BlockUnit* units, const BlockUnit* host_units, uint32_t n_units,
                            bool to_far, hipStream_t s, bool* launched) {
  *launched = false;
  if (n_units == 0 || n_units > kMaxRowUnits) return PF_OK;
  RowEnds ends;
  uint64_t rows = 0, max_frag = 0;
  uint32_t max_seg = 0;
  for (uint32_t k = 0; k < kMaxRowUnits; ++k) {
    if (k < n_units) {
      const BlockUnit& u = host_units[k];
      if (u.n_seg != 1 && u.n_seg != 2) {
        return fail(PF_ERR_INVALID_ARGUMENT, "tile launch: %u segments per block", u.n_seg);
      }
      rows += u.n_blocks;
      max_frag = max_frag < u.frag_bytes ? u.frag_bytes : max_frag;
      max_seg = max_seg < u.n_seg ? u.n_seg : max_seg;
    }
    ends.end[k] = k + 1 < n_units ? static_cast<uint32_t>(rows) : UINT32_MAX;
  }
  constexpr uint64_t kTile = kTileLanes * 16;
  const uint64_t gx = (max_frag + kTile - 1) / kTile;
  if (rows == 0 || max_frag == 0) {
    *launched = true;
    return PF_OK;
  }
  // Rows beyond one grid extent go into further chunks of equal length along grid.z.
  const uint64_t chunks = (rows + kMaxTileBlocks - 1) / kMaxTileBlocks;
  const uint64_t gy = (rows + chunks - 1) / chunks;
  if (chunks * max_seg > kMaxTileBlocks || rows >= 0xFFFFFFFFull || gx > 0x7FFFFFFFull) {
    return PF_OK;  // the caller takes another form
  }
  dim3 grid(static_cast<uint32_t>(gx), static_cast<uint32_t>(gy),
            static_cast<uint32_t>(chunks * max_seg));
  dim3 block(kTileLanes, 1, 1);
  if (max_seg == 2) {
    if (to_far) {
      hipLaunchKernelGGL((block_tiles_rows_kernel<kTileLanes, true, 2>), grid, block, 0, s, units, ends);
    } else {
      hipLaunchKernelGGL((block_tiles_rows_kernel<kTileLanes, false, 2>), grid, block, 0, s, units, ends);
    }
  } else if (to_far) {
    hipLaunchKernelGGL((block_tiles_rows_kernel<kTileLanes, true, 1>), grid, block, 0, s, units, ends);
  } else {
    hipLaunchKernelGGL((block_tiles_rows_kernel<kTileLanes, false, 1>), grid, block, 0, s, units, ends);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "block_tiles_rows_kernel launch");
  *launched = true;
  return PF_OK;
}

int launch_block_tiles(const BlockUnit* units, uint32_t n_units, uint32_t max_blocks,
                       uint64_t max_frag_bytes, uint32_t max_seg, bool to_far, hipStream_t s) {
  if (n_units == 0 || max_blocks == 0 || max_frag_bytes == 0) return PF_OK;
  if (max_seg != 1 && max_seg != 2) {
    return fail(PF_ERR_INVALID_ARGUMENT, "tile launch: %u segments per block", max_seg);
  }
  constexpr uint64_t kTile = kTileLanes * 16;
  const uint64_t gx = (max_frag_bytes + kTile - 1) / kTile;
  if (n_units > kMaxTileUnits || max_blocks > kMaxTileBlocks || gx > 0x7FFFFFFFull) {
    return fail(PF_ERR_INVALID_ARGUMENT,
                "tile launch out of range: %u units, %u blocks, %llu-byte fragments", n_units,
                max_blocks, static_cast<unsigned long long>(max_frag_bytes));
  }
  // A launch over several units (the layers of page-first pages) makes the
  // units the inner grid dimension: the staging side is then walked page after
  // page and every cache in ascending position order.  Measured on the
  // DeepSeek-V3 page-first shape (61 units x 119 pages per launch): gather
  // 5.3 -> 5.9 TB/s, scatter 5.5 -> 6.2 TB/s against positions-inner.
  // A few units of equal length (page packing of a model with few layers) keep
  // the order of a single unit, one (unit, segment) after the other: with 2-4
  // units per launch that form measured 1-2 % faster than units-inner (Llama
  // shape, three layers per launch: 6.10 against 6.04 TB/s; fp8 shape, four:
  // 6.18 against 6.10).  Staging fills of up to eight units of unlike lengths
  // do not come here: launch_block_tiles_rows.
  constexpr uint32_t kUnitsInnerFrom = 9;
  const bool units_inner = n_units >= kUnitsInnerFrom;
  const uint32_t unit_segs = max_seg * n_units;
  dim3 grid(static_cast<uint32_t>(gx), units_inner ? unit_segs : max_blocks,
            units_inner ? max_blocks : unit_segs);
  dim3 block(kTileLanes, 1, 1);
#define PF_LAUNCH_TILES(TO_FAR_, SEGS_, INNER_)                                                \
  hipLaunchKernelGGL((block_tiles_kernel<kTileLanes, TO_FAR_, SEGS_, INNER_>), grid, block, 0, s, \
                     units)
  if (units_inner) {
    if (max_seg == 2) {
      if (to_far) {
        PF_LAUNCH_TILES(true, 2, true);
      } else {
        PF_LAUNCH_TILES(false, 2, true);
      }
    } else {
      if (to_far) {
        PF_LAUNCH_TILES(true, 1, true);
      } else {
        PF_LAUNCH_TILES(false, 1, true);
      }
    }
  } else if (max_seg == 2) {
    if (to_far) {
      PF_LAUNCH_TILES(true, 2, false);
    } else {
      PF_LAUNCH_TILES(false, 2, false);
    }
  } else {
    if (to_far) {
      PF_LAUNCH_TILES(true, 1, false);
    } else {
      PF_LAUNCH_TILES(false, 1, false);
    }
  }
#undef PF_LAUNCH_TILES
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "block_tiles_kernel launch");
  return PF_OK;
}

}  // namespace pf

// The two words of the stream-concurrency probe ([0] the posted word, [1] what
// the waiter saw) live in the library's device image: a probe allocates and
// frees nothing, so it never waits for unrelated work on the device (hipFree
// synchronises the whole device).
static __device__ __align__(256) uint32_t probe_words[2];

namespace pf {

namespace {
constexpr int kProbeMaxDevices = 64;
std::mutex g_probe_mu;  // one probe at a time: they share the two words
uint32_t* g_probe_ptr[kProbeMaxDevices] = {};

int probe_words_on_current_device(uint32_t** out) {
  int device = -1;
  PF_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kProbeMaxDevices) {
    return fail(PF_ERR_INVALID_ARGUMENT, "device %d is beyond the %d the probe supports", device,
                kProbeMaxDevices);
  }
  if (g_probe_ptr[device] == nullptr) {
    void* ptr = nullptr;
    PF_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(probe_words)));
    g_probe_ptr[device] = static_cast<uint32_t*>(ptr);
  }
  *out = g_probe_ptr[device];
  return PF_OK;
}
}  // namespace

int streams_run_concurrently(hipStream_t a, hipStream_t b, bool* out) {
  *out = false;
  std::lock_guard<std::mutex> lock(g_probe_mu);
  uint32_t* words = nullptr;
  int st = probe_words_on_current_device(&words);
  if (st != PF_OK) return st;
  uint32_t seen = 0;
  // Cleared on `a` and waited for there: no other stream of the device is touched.
  hipError_t e = hipMemsetAsync(words, 0, 2 * sizeof(uint32_t), a);
  if (e == hipSuccess) e = hipStreamSynchronize(a);
  if (e == hipSuccess) {
    constexpr uint64_t kMaxTicks = 200000;  // 2 ms of the 100 MHz clock
    hipLaunchKernelGGL(probe_wait_kernel, dim3(1), dim3(64), 0, a, words, words + 1, kMaxTicks);
    hipLaunchKernelGGL(probe_post_kernel, dim3(1), dim3(64), 0, b, words);
    e = hipGetLastError();
  }
  // Wait for both whatever was launched: the next probe reuses the words.
  const hipError_t ea = hipStreamSynchronize(a);
  const hipError_t eb = hipStreamSynchronize(b);
  if (e == hipSuccess) e = ea != hipSuccess ? ea : eb;
  if (e == hipSuccess) e = hipMemcpyAsync(&seen, words + 1, sizeof(seen), hipMemcpyDeviceToHost, a);
  if (e == hipSuccess) e = hipStreamSynchronize(a);
  if (e != hipSuccess) st = fail_hip(e, "stream concurrency probe");
  *out = seen != 0;
  return st;
}

int launch_plain_copy(void* dst, const void* src, uint64_t bytes, int unroll, hipStream_t s) {
  if (bytes == 0) return PF_OK;
  if ((bytes & 15ull) != 0 || (reinterpret_cast<uint64_t>(dst) & 15ull) != 0 ||
      (reinterpret_cast<uint64_t>(src) & 15ull) != 0) {
    return fail(PF_ERR_INVALID_ARGUMENT, "plain copy needs 16-byte aligned pointers and size");
  }
  if (unroll == 0) {
    constexpr uint64_t kTile = kTileLanes * 16;
    const uint64_t n = (bytes + kTile - 1) / kTile;
    // Exactly one workgroup per tile, like the gather / scatter grids: a
    // yardstick that launched idle workgroups (a 65 536-wide grid rounded up to
    // whole rows: 18 % of them for a 327 MB copy) read 4 % low.
    if (n > 0x7FFFFFFFull) return fail(PF_ERR_INVALID_ARGUMENT, "plain copy too large");
    hipLaunchKernelGGL(plain_tiles_kernel<kTileLanes>, dim3(static_cast<uint32_t>(n), 1, 1),
                       dim3(kTileLanes, 1, 1), 0, s, reinterpret_cast<uint64_t>(dst),
                       reinterpret_cast<uint64_t>(src), bytes);
    hipError_t e0 = hipGetLastError();
    if (e0 != hipSuccess) return fail_hip(e0, "plain_tiles_kernel launch");
    return PF_OK;
  }
  const uint64_t tile = tile_bytes(unroll);
  uint64_t tiles = (bytes + tile - 1) / tile;
  uint32_t gx = static_cast<uint32_t>(tiles < kMaxGridX ? tiles : kMaxGridX);
  dim3 grid(gx, 1, 1), block(kLanes, 1, 1);
  const uint64_t d = reinterpret_cast<uint64_t>(dst);
  const uint64_t c = reinterpret_cast<uint64_t>(src);
  switch (unroll) {
    case 1: hipLaunchKernelGGL(plain_copy_kernel<1>, grid, block, 0, s, d, c, bytes); break;
    case 2: hipLaunchKernelGGL(plain_copy_kernel<2>, grid, block, 0, s, d, c, bytes); break;
    case 4: hipLaunchKernelGGL(plain_copy_kernel<4>, grid, block, 0, s, d, c, bytes); break;
    case 8: hipLaunchKernelGGL(plain_copy_kernel<8>, grid, block, 0, s, d, c, bytes); break;
    default: return fail(PF_ERR_INVALID_ARGUMENT, "unsupported tile unroll %d", unroll);
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "plain_copy_kernel launch");
  return PF_OK;
}

namespace {
// Grid of a descriptor-copy launch: x over descriptors, y over the tiles of the
// largest one.  The kernels stride in both dimensions, so any grid covers the
// batch; `max_workgroups` (0 = no cap) bounds the whole launch.
dim3 desc_copy_grid(uint64_t n, uint64_t max_size, uint32_t max_workgroups) {
  constexpr uint64_t kTile = tile_bytes(kDescUnroll);
  uint64_t gx = n < kMaxGridX ? n : kMaxGridX;
  uint64_t gy = (max_size + kTile - 1) / kTile;
  if (gy < 1) gy = 1;
  if (gy > 64) gy = 64;
  if (max_workgroups != 0) {
    while (gx * gy > max_workgroups && gy > 1) gy >>= 1;
    if (gx * gy > max_workgroups) gx = max_workgroups / gy ? max_workgroups / gy : 1;
  }
  // Keep the launch to a few million workgroups; a smaller grid only means
  // more iterations per workgroup.
  while (gx * gy > (1ull << 22) && gy > 1) gy >>= 1;
  return dim3(static_cast<uint32_t>(gx), static_cast<uint32_t>(gy), 1);
}
}  // namespace

int launch_desc_copy(const uint64_t* table, uint64_t n, uint64_t max_size, hipStream_t s,
                     uint32_t max_workgroups) {
  if (n == 0) return PF_OK;
  const dim3 grid = desc_copy_grid(n, max_size, max_workgroups), block(kLanes, 1, 1);
  hipLaunchKernelGGL(desc_copy_kernel<kDescUnroll>, grid, block, 0, s, table,
                     static_cast<uint32_t>(n));
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail_hip(e, "desc_copy_kernel launch");
  return PF_OK;
}

}  // namespace pf

// ---------------------------------------------------------------------------
// Descriptor copy that allocates nothing
// ---------------------------------------------------------------------------
//
// The kernel backend keeps its descriptor table in device memory it allocates
// (and grows) on demand.  Callers that must not allocate get the same copy with
// the table in a fixed array that is part of the library's device image.  Every
// GPU the library runs on holds its own copy of the array, at its own address,
// until the process ends, and every call on a GPU shares it.  Nothing in it has
// to start at zero: a call overwrites rows [0, n) before its kernel reads
// exactly those rows.  Calls are ordered among themselves: the upload and the
// launch of a call are issued under one lock, and the upload waits (on the
// device) for an event recorded behind the previous call's kernel, whichever
// stream that ran on, so a call never overwrites rows a kernel is still
// reading.  Calls on different streams of one GPU therefore run one after the
// other; that is the price of the single table.

// Most descriptors one call takes: 32768 x 48 bytes = 1.5 MiB per GPU.
#define PF_NOALLOC_MAX_DESCS 32768u

static __device__ __align__(256) unsigned char scratch[PF_NOALLOC_MAX_DESCS * sizeof(pf_copy_desc)];

namespace {

constexpr int kNoAllocMaxDevices = 64;
// Same rule as the kernel backend: the host link wants few requesters, 16
// workgroups when the average fragment fills a 16 KiB tile, up to 64 below.
uint32_t noalloc_workgroups(uint64_t total_bytes, uint64_t n) {
  constexpr uint64_t kTile = 16384;
  const uint64_t avg = total_bytes / n ? total_bytes / n : 1;
  if (avg >= kTile) return 16;
  const uint64_t scaled = 16 * ((kTile + avg - 1) / avg);
  return static_cast<uint32_t>(scaled < 64 ? scaled : 64);
}

// Per device: the table's address, the event behind the last call's kernel, and
// whether there has been a call.  Set up on a device's first call (address and
// event are host-side objects: no device or pinned memory is allocated).
struct NoAllocDevice {
  void* table = nullptr;
  hipEvent_t last_done = nullptr;
  bool used = false;
};
std::mutex g_scratch_mu;
NoAllocDevice g_noalloc[kNoAllocMaxDevices];

// Device address of `scratch` on the current device.  The array's name is only
// a host-side handle for the symbol; the address comes from the runtime, once
// per device, and is what every later use takes.  g_scratch_mu held.
int noalloc_on_current_device(NoAllocDevice** out) {
  int device = -1;
  PF_HIP(hipGetDevice(&device));
  if (device < 0 || device >= kNoAllocMaxDevices) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT, "device %d is beyond the %d this call supports",
                    device, kNoAllocMaxDevices);
  }
  NoAllocDevice& d = g_noalloc[device];
  if (d.table == nullptr) {
    void* ptr = nullptr;
    PF_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)));
    if (ptr == nullptr) {
      return pf::fail(PF_ERR_DEVICE_INIT, "hipGetSymbolAddress(scratch) returned a null address");
    }
    hipEvent_t done = nullptr;
    PF_HIP(hipEventCreateWithFlags(&done, hipEventDisableTiming));
    d.last_done = done;
    d.table = ptr;
  }
  *out = &d;
  return PF_OK;
}

}  // namespace

extern "C" int pf_desc_copy_noalloc(const pf_copy_desc* copies, uint64_t n, int host_is_src,
                                    pf_stream_t s) {
  if (n == 0) return PF_OK;
  PF_REQUIRE_PTR(copies);
  if (n > PF_NOALLOC_MAX_DESCS) {
    return pf::fail(PF_ERR_INVALID_ARGUMENT,
                    "pf_desc_copy_noalloc takes at most %u descriptors per call, got %llu "
                    "(split the batch, or use pf_backend_h2d / pf_backend_d2h)",
                    PF_NOALLOC_MAX_DESCS, static_cast<unsigned long long>(n));
  }
  uint64_t max_size = 0, total_size = 0;
  for (uint64_t i = 0; i < n; ++i) {
    const pf_copy_desc& c = copies[i];
    total_size += c.size;
    if (c.size != 0 && (c.device == 0 || c.host_device == 0)) {
      // The kernel dereferences both addresses; a null one would fault the GPU.
      return pf::fail(PF_ERR_INVALID_ARGUMENT,
                      "descriptor %llu: the copy kernel needs a device address and a "
                      "device-visible host address",
                      static_cast<unsigned long long>(i));
    }
    if (c.size > max_size) max_size = c.size;
  }
  if (max_size == 0) return PF_OK;
  // Upload and launch under one lock: two threads cannot interleave their rows.
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  NoAllocDevice* dev = nullptr;
  int st = noalloc_on_current_device(&dev);
  if (st != PF_OK) return st;
  hipStream_t stream = pf::native(s);
  // The previous call's kernel may still be reading the table, on this stream
  // or another: this call's upload waits for it on the device.
  if (dev->used) PF_HIP(hipStreamWaitEvent(stream, dev->last_done, 0));
  // The caller's array is the table: one copy.  From pinned memory it is
  // asynchronous; from pageable memory the runtime stages it before returning.
  PF_HIP(hipMemcpyAsync(dev->table, copies, n * sizeof(pf_copy_desc), hipMemcpyHostToDevice, stream));
  const dim3 grid = pf::desc_copy_grid(n, max_size, noalloc_workgroups(total_size, n)), block(pf::kLanes, 1, 1);
  const pf_copy_desc* rows = static_cast<const pf_copy_desc*>(dev->table);
  if (host_is_src) {
    hipLaunchKernelGGL((pf::desc48_copy_kernel<pf::kDescUnroll, true>), grid, block, 0, stream, rows,
                       static_cast<uint32_t>(n));
  } else {
    hipLaunchKernelGGL((pf::desc48_copy_kernel<pf::kDescUnroll, false>), grid, block, 0, stream,
                       rows, static_cast<uint32_t>(n));
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return pf::fail_hip(e, "desc48_copy_kernel launch");
  PF_HIP(hipEventRecord(dev->last_done, stream));
  dev->used = true;
  return PF_OK;
}

extern "C" uint64_t pf_desc_copy_noalloc_max(void) { return PF_NOALLOC_MAX_DESCS; }
