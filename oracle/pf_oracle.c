/*
 * pf_oracle.c — CPU restatement of the reference's KV block transfer path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (libpegahip, the
 * pegaflow_amd package) may link, import or call this file.  It is used by
 * tests/, by the smoke check and by the cpu_baseline leg of bench.py, as the
 * checker — never as the thing measured or shipped.
 *
 * Each function restates one piece of novitalabs/pegaflow and cites the file
 * and lines it follows.  "Device" memory is ordinary host memory here: a
 * device address is simply a pointer into a host-resident cache image.
 *
 * What pins it (see tests/test_oracle_*.py): the reference's own unit-test
 * vectors for layout.rs, memcpy.rs and instance/tests.rs; a literal emulation
 * of the reference's copy kernel loop nest; and an independent numpy
 * fancy-index gather/scatter on small random inputs.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ORC_OK 0
#define ORC_ERR 1

typedef struct orc_layout {
  uint64_t data_ptr;
  uint64_t size_bytes;
  uint64_t num_blocks;
  uint64_t block_stride_bytes;
  uint64_t segment_bytes;
  uint64_t segments;
  uint64_t padded_segment_bytes;
  uint64_t kv_stride_bytes; /* meaningful when split */
  int32_t split;
  int32_t pad_;
} orc_layout;

typedef struct orc_desc {
  uint64_t device;
  uint64_t host;
  uint64_t host_device;
  uint64_t size;
  uint64_t device_allocation;
  uint64_t host_allocation;
} orc_desc;

typedef struct orc_range {
  uint64_t device;
  uint64_t host;
  uint64_t size;
} orc_range;

static int seterr(char* err, size_t cap, const char* msg) {
  if (err && cap) snprintf(err, cap, "%s", msg);
  return ORC_ERR;
}

static int mul_u64(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_mul_overflow(a, b, r); }
static int add_u64(uint64_t a, uint64_t b, uint64_t* r) { return __builtin_add_overflow(a, b, r); }

/* ----------------------------------------------------------------------- */
/* layout.rs:196-229 check_bounds + check_split_segments_disjoint           */
/* ----------------------------------------------------------------------- */

static int orc_check_disjoint(const orc_layout* l, char* err, size_t cap) {
  /* layout.rs:206-226 */
  uint64_t max_block_distance = l->num_blocks - 1;
  uint64_t nearest = l->kv_stride_bytes / l->block_stride_bytes;
  uint64_t cand[2];
  cand[0] = nearest;
  cand[1] = nearest == UINT64_MAX ? UINT64_MAX : nearest + 1; /* saturating_add */
  for (int i = 0; i < 2; ++i) {
    uint64_t distance = cand[i];
    if (distance == 0 || distance > max_block_distance) continue;
    uint64_t dist_bytes;
    if (mul_u64(distance, l->block_stride_bytes, &dist_bytes))
      return seterr(err, cap, "memory layout overflow");
    uint64_t gap = l->kv_stride_bytes > dist_bytes ? l->kv_stride_bytes - dist_bytes
                                                    : dist_bytes - l->kv_stride_bytes;
    if (gap < l->segment_bytes) {
      char buf[160];
      snprintf(buf, sizeof buf, "kv_stride_bytes %llu overlaps blocks %llu apart",
               (unsigned long long)l->kv_stride_bytes, (unsigned long long)distance);
      return seterr(err, cap, buf);
    }
  }
  return ORC_OK;
}

static int orc_check_bounds(const orc_layout* l, char* err, size_t cap) {
  /* layout.rs:164-204 */
  char buf[200];
  uint64_t end, t;
  if (!l->split) {
    uint64_t block_bytes = l->segment_bytes * l->segments;
    if (l->block_stride_bytes < block_bytes) {
      snprintf(buf, sizeof buf, "block_stride %llu must be >= block_bytes %llu: blocks would overlap",
               (unsigned long long)l->block_stride_bytes, (unsigned long long)block_bytes);
      return seterr(err, cap, buf);
    }
    if (mul_u64(l->num_blocks - 1, l->block_stride_bytes, &t) || add_u64(t, block_bytes, &end))
      return seterr(err, cap, "memory layout overflow");
  } else {
    if (l->block_stride_bytes < l->segment_bytes) {
      snprintf(buf, sizeof buf,
               "block_stride %llu must be >= segment_bytes %llu: blocks would overlap",
               (unsigned long long)l->block_stride_bytes, (unsigned long long)l->segment_bytes);
      return seterr(err, cap, buf);
    }
    if (orc_check_disjoint(l, err, cap)) return ORC_ERR;
    uint64_t last_segment_end;
    if (mul_u64(l->num_blocks - 1, l->block_stride_bytes, &t) ||
        add_u64(t, l->segment_bytes, &last_segment_end) ||
        add_u64(l->kv_stride_bytes, last_segment_end, &end))
      return seterr(err, cap, "memory layout overflow");
  }
  if (end > l->size_bytes) {
    snprintf(buf, sizeof buf, "registered memory too small: need %llu bytes, got %llu",
             (unsigned long long)end, (unsigned long long)l->size_bytes);
    return seterr(err, cap, buf);
  }
  return ORC_OK;
}

/* layout.rs:73-130 KVCacheLayout::new */
int orc_layout_new(uint64_t data_ptr, uint64_t size_bytes, uint64_t num_blocks,
                   uint64_t segment_bytes, uint64_t kv_stride_bytes, uint64_t segments,
                   orc_layout* out, char* err, size_t cap) {
  char buf[240];
  uint64_t t, block_bytes;
  if (data_ptr == 0) return seterr(err, cap, "data_ptr must not be null");
  if (size_bytes == 0) return seterr(err, cap, "size_bytes must be > 0");
  if (segment_bytes == 0 || num_blocks == 0 || segments == 0)
    return seterr(err, cap, "segment_bytes, num_blocks, and segments must be non-zero");
  if (add_u64(data_ptr, size_bytes, &t))
    return seterr(err, cap, "data_ptr + size_bytes overflows the address space");
  if (mul_u64(segment_bytes, segments, &block_bytes)) return seterr(err, cap, "block size overflow");

  int split = 0;
  if (segments == 1) {
    split = 0;
  } else if (kv_stride_bytes == 0) {
    return seterr(err, cap, "kv_stride_bytes must be > 0 when segments > 1");
  } else if (kv_stride_bytes < segment_bytes) {
    snprintf(buf, sizeof buf, "kv_stride_bytes %llu < segment_bytes %llu: segments would overlap",
             (unsigned long long)kv_stride_bytes, (unsigned long long)segment_bytes);
    return seterr(err, cap, buf);
  } else if (kv_stride_bytes == segment_bytes) {
    split = 0;
  } else if (segments == 2) {
    split = 1;
  } else {
    snprintf(buf, sizeof buf,
             "split layout (kv_stride_bytes %llu > segment_bytes %llu) supports exactly 2 "
             "segments, got %llu",
             (unsigned long long)kv_stride_bytes, (unsigned long long)segment_bytes,
             (unsigned long long)segments);
    return seterr(err, cap, buf);
  }
  orc_layout l;
  memset(&l, 0, sizeof l);
  l.data_ptr = data_ptr;
  l.size_bytes = size_bytes;
  l.num_blocks = num_blocks;
  l.block_stride_bytes = split ? segment_bytes : block_bytes;
  l.segment_bytes = segment_bytes;
  l.segments = segments;
  l.padded_segment_bytes = segment_bytes;
  l.kv_stride_bytes = split ? kv_stride_bytes : 0;
  l.split = split;
  if (orc_check_bounds(&l, err, cap)) return ORC_ERR;
  *out = l;
  return ORC_OK;
}

/* layout.rs:140-153 with_block_stride */
int orc_layout_with_block_stride(orc_layout* l, uint64_t stride, char* err, size_t cap) {
  char buf[200];
  uint64_t min_stride = l->split ? l->segment_bytes : l->segment_bytes * l->segments;
  if (stride < min_stride) {
    snprintf(buf, sizeof buf, "block_stride %llu must be >= %llu: blocks would overlap",
             (unsigned long long)stride, (unsigned long long)min_stride);
    return seterr(err, cap, buf);
  }
  orc_layout c = *l;
  c.block_stride_bytes = stride;
  if (orc_check_bounds(&c, err, cap)) return ORC_ERR;
  *l = c;
  return ORC_OK;
}

/* layout.rs:157-160 with_ssd_padding (next_multiple_of) */
void orc_layout_with_ssd_padding(orc_layout* l, uint64_t alignment) {
  uint64_t q = (l->segment_bytes + alignment - 1) / alignment;
  l->padded_segment_bytes = q * alignment;
}

/* layout.rs:231-255 block_copies */
int orc_block_copies(const orc_layout* l, uint64_t block_idx, uint64_t addr[2], uint64_t bytes[2],
                     int* n, char* err, size_t cap) {
  if (block_idx >= l->num_blocks) {
    char buf[120];
    snprintf(buf, sizeof buf, "block %llu out of range (%llu blocks)",
             (unsigned long long)block_idx, (unsigned long long)l->num_blocks);
    return seterr(err, cap, buf);
  }
  uint64_t base = l->data_ptr + block_idx * l->block_stride_bytes;
  if (l->split) {
    *n = 2;
    addr[0] = base;
    bytes[0] = l->segment_bytes;
    addr[1] = base + l->kv_stride_bytes;
    bytes[1] = l->segment_bytes;
  } else {
    *n = 1;
    addr[0] = base;
    bytes[0] = l->segment_bytes * l->segments;
    addr[1] = 0;
    bytes[1] = 0;
  }
  return ORC_OK;
}

/* ----------------------------------------------------------------------- */
/* transfer/memcpy.rs:25-55 merge                                           */
/* ----------------------------------------------------------------------- */

uint64_t orc_merge(const orc_desc* copies, uint64_t n, orc_range* out) {
  uint64_t n_out = 0;
  uint64_t i = 0;
  while (i < n) {
    orc_desc start = copies[i];
    uint64_t size = start.size;
    uint64_t j = i + 1;
    while (j < n) {
      orc_desc next = copies[j];
      int same_allocations = start.device_allocation == next.device_allocation &&
                             start.host_allocation == next.host_allocation;
      int device_contiguous = start.device + size == next.device;
      int host_contiguous = start.host + size == next.host;
      if (same_allocations && device_contiguous && host_contiguous) {
        size += next.size;
        j += 1;
      } else {
        break;
      }
    }
    out[n_out].device = start.device;
    out[n_out].host = start.host;
    out[n_out].size = size;
    n_out += 1;
    i = j;
  }
  return n_out;
}

/* ----------------------------------------------------------------------- */
/* gpu_worker.rs:353-423 build_copy_descs                                   */
/*                                                                          */
/* A layer's blocks are given as parallel arrays: device slot, then for the */
/* host image up to two segments (host address, device-visible address,     */
/* allocation id); seg1_host[i] == 0 marks a single-segment host block.     */
/* ----------------------------------------------------------------------- */

typedef struct orc_layer {
  orc_layout layout;
  const uint64_t* block_idx;
  const uint64_t* seg0_host;
  const uint64_t* seg0_dev;
  const uint64_t* seg0_alloc;
  const uint64_t* seg1_host; /* may be NULL */
  const uint64_t* seg1_dev;
  const uint64_t* seg1_alloc;
  const uint64_t* host_offset; /* may be NULL = all zero */
  uint64_t n_blocks;
} orc_layer;

int orc_build_copy_descs(const orc_layer* layers, uint64_t n_layers, orc_desc* out, uint64_t cap_out,
                         uint64_t* n_out, uint64_t* total_bytes, uint64_t* bad_layer, char* err,
                         size_t cap) {
  uint64_t n = 0, total = 0;
  for (uint64_t li = 0; li < n_layers; ++li) {
    const orc_layer* L = &layers[li];
    for (uint64_t b = 0; b < L->n_blocks; ++b) {
      uint64_t addr[2], bytes[2];
      int nc = 0;
      if (orc_block_copies(&L->layout, L->block_idx[b], addr, bytes, &nc, err, cap)) {
        if (bad_layer) *bad_layer = li;
        return ORC_ERR;
      }
      uint64_t off = L->host_offset ? L->host_offset[b] : 0;
      if (nc == 2) {
        uint64_t k_host = L->seg0_host[b] + off;
        uint64_t k_dev = L->seg0_dev[b] + off;
        int has_v = L->seg1_host && L->seg1_host[b] != 0;
        /* gpu_worker.rs:373-379: no segment 1 => V follows K */
        uint64_t v_host = has_v ? L->seg1_host[b] + off : k_host + bytes[0];
        uint64_t v_dev = has_v ? L->seg1_dev[b] + off : k_dev + bytes[0];
        uint64_t v_alloc = has_v ? L->seg1_alloc[b] : L->seg0_alloc[b];
        if (n + 2 > cap_out) return seterr(err, cap, "descriptor buffer too small");
        out[n++] = (orc_desc){addr[0], k_host, k_dev, bytes[0], li, L->seg0_alloc[b]};
        out[n++] = (orc_desc){addr[1], v_host, v_dev, bytes[1], li, v_alloc};
        total += bytes[0] + bytes[1];
      } else {
        if (n + 1 > cap_out) return seterr(err, cap, "descriptor buffer too small");
        out[n++] = (orc_desc){addr[0], L->seg0_host[b] + off, L->seg0_dev[b] + off, bytes[0], li,
                              L->seg0_alloc[b]};
        total += bytes[0];
      }
    }
  }
  *n_out = n;
  if (total_bytes) *total_bytes = total;
  return ORC_OK;
}

/* ----------------------------------------------------------------------- */
/* Executors.                                                               */
/* transfer/memcpy.rs:57-102: one copy per merged range;                    */
/* transfer/kernel.rs:79-135: dst/src chosen by direction, one copy per     */
/* descriptor.  Both are `memcpy(dst, src, size)` per range.                */
/* ----------------------------------------------------------------------- */

typedef struct orc_job {
  const orc_range* ranges;
  uint64_t begin, end;
  int host_is_src;
} orc_job;

static void* orc_worker(void* arg) {
  orc_job* j = (orc_job*)arg;
  for (uint64_t i = j->begin; i < j->end; ++i) {
    const orc_range* r = &j->ranges[i];
    void* dev = (void*)(uintptr_t)r->device;
    void* host = (void*)(uintptr_t)r->host;
    if (j->host_is_src)
      memcpy(dev, host, r->size);
    else
      memcpy(host, dev, r->size);
  }
  return NULL;
}

/* Copy every range; ranges are split into `threads` contiguous chunks of
 * equal count (a static-chunk thread pool). */
static void orc_run_ranges(const orc_range* ranges, uint64_t n, int host_is_src, int threads) {
  if (threads <= 1 || n < 2) {
    orc_job j = {ranges, 0, n, host_is_src};
    orc_worker(&j);
    return;
  }
  if ((uint64_t)threads > n) threads = (int)n;
  pthread_t* tids = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
  orc_job* jobs = (orc_job*)malloc(sizeof(orc_job) * (size_t)threads);
  uint64_t per = (n + (uint64_t)threads - 1) / (uint64_t)threads;
  int started = 0;
  for (int t = 0; t < threads; ++t) {
    uint64_t b = per * (uint64_t)t;
    if (b >= n) break;
    uint64_t e = b + per < n ? b + per : n;
    jobs[t] = (orc_job){ranges, b, e, host_is_src};
    pthread_create(&tids[t], NULL, orc_worker, &jobs[t]);
    started++;
  }
  for (int t = 0; t < started; ++t) pthread_join(tids[t], NULL);
  free(tids);
  free(jobs);
}

/* direct backend: merge, then one memcpy per range */
void orc_exec_direct(const orc_desc* copies, uint64_t n, int host_is_src, int threads) {
  if (n == 0) return;
  orc_range* ranges = (orc_range*)malloc(sizeof(orc_range) * n);
  uint64_t m = orc_merge(copies, n, ranges);
  orc_run_ranges(ranges, m, host_is_src, threads);
  free(ranges);
}

/* kernel backend: one memcpy per descriptor, host side through host_device */
void orc_exec_kernel(const orc_desc* copies, uint64_t n, int host_is_src, int threads) {
  if (n == 0) return; /* kernel.rs:85-87 */
  orc_range* ranges = (orc_range*)malloc(sizeof(orc_range) * n);
  for (uint64_t i = 0; i < n; ++i) {
    ranges[i].device = copies[i].device;
    ranges[i].host = copies[i].host_device;
    ranges[i].size = copies[i].size;
  }
  orc_run_ranges(ranges, n, host_is_src, threads);
  free(ranges);
}

/* Literal emulation of the reference copy kernel's loop nest
 * (transfer/kernel.rs:25-46) for a given grid and block size: every
 * (block, thread) executes its share of 16-byte words and tail bytes, or the
 * byte loop when either address is not 16-byte aligned.  Slow; for small
 * inputs, to show the kernel is `memcpy` per descriptor. */
void orc_emulate_batch_copy_kernel(const uint64_t* descs, int n, unsigned grid_dim,
                                   unsigned block_dim) {
  for (unsigned block = 0; block < grid_dim; ++block) {
    for (unsigned thread = 0; thread < block_dim; ++thread) {
      for (int i = (int)block; i < n; i += (int)grid_dim) {
        char* dst = (char*)(uintptr_t)descs[3 * i + 0];
        const char* src = (const char*)(uintptr_t)descs[3 * i + 1];
        unsigned long long size = descs[3 * i + 2];
        if ((((unsigned long long)(uintptr_t)dst | (unsigned long long)(uintptr_t)src) & 15ULL) ==
            0ULL) {
          unsigned long long n16 = size >> 4;
          for (unsigned long long j = thread; j < n16; j += block_dim)
            memcpy(dst + 16 * j, src + 16 * j, 16);
          for (unsigned long long j = (n16 << 4) + thread; j < size; j += block_dim)
            dst[j] = src[j];
        } else {
          for (unsigned long long j = thread; j < size; j += block_dim) dst[j] = src[j];
        }
      }
    }
  }
}

/* ----------------------------------------------------------------------- */
/* instance.rs:107-162 build_page_layout                                    */
/*                                                                          */
/* Worker layer-id sets arrive flattened: set w is                          */
/* set_ids[set_off[w] .. set_off[w+1]) (any order, duplicates ignored).     */
/* Outputs are indexed by layer id, shard sizes by shard id.                */
/* Returns 0, or 1 = overlap ("claimed by shards"), 2 = gap ("no shard      */
/* owner"); *bad_layer names the offending layer.                           */
/* ----------------------------------------------------------------------- */

static int cmp_u64(const void* a, const void* b) {
  uint64_t x = *(const uint64_t*)a, y = *(const uint64_t*)b;
  return x < y ? -1 : x > y;
}

int orc_build_page_layout(const uint64_t* set_ids, const uint64_t* set_off, uint64_t n_sets,
                          uint64_t n_layers, const uint64_t* padded_bytes, uint64_t* layer_shard,
                          uint64_t* layer_offsets, uint64_t* layer_bytes, uint64_t* shard_page_sizes,
                          uint64_t* n_shards_out, uint64_t* bad_layer, uint64_t* bad_shard_a,
                          uint64_t* bad_shard_b) {
  /* Normalise every set to sorted unique ids (BTreeSet). */
  uint64_t** sets = (uint64_t**)calloc(n_sets ? n_sets : 1, sizeof(uint64_t*));
  uint64_t* lens = (uint64_t*)calloc(n_sets ? n_sets : 1, sizeof(uint64_t));
  for (uint64_t w = 0; w < n_sets; ++w) {
    uint64_t len = set_off[w + 1] - set_off[w];
    sets[w] = (uint64_t*)malloc(sizeof(uint64_t) * (len ? len : 1));
    memcpy(sets[w], set_ids + set_off[w], sizeof(uint64_t) * len);
    qsort(sets[w], len, sizeof(uint64_t), cmp_u64);
    uint64_t u = 0;
    for (uint64_t i = 0; i < len; ++i)
      if (i == 0 || sets[w][i] != sets[w][i - 1]) sets[w][u++] = sets[w][i];
    lens[w] = u;
  }
  /* Distinct sets become shards, in first-seen order... */
  uint64_t* shard_of = (uint64_t*)malloc(sizeof(uint64_t) * (n_sets ? n_sets : 1));
  uint64_t n_shards = 0;
  for (uint64_t w = 0; w < n_sets; ++w) {
    int seen = 0;
    for (uint64_t s = 0; s < n_shards; ++s) {
      uint64_t o = shard_of[s];
      if (lens[o] == lens[w] && memcmp(sets[o], sets[w], sizeof(uint64_t) * lens[w]) == 0) {
        seen = 1;
        break;
      }
    }
    if (!seen) shard_of[n_shards++] = w;
  }
  /* ...then ordered by minimum layer id (stable, empty set last). */
  for (uint64_t a = 1; a < n_shards; ++a) {
    uint64_t w = shard_of[a];
    uint64_t key = lens[w] ? sets[w][0] : UINT64_MAX;
    uint64_t b = a;
    while (b > 0) {
      uint64_t pw = shard_of[b - 1];
      uint64_t pkey = lens[pw] ? sets[pw][0] : UINT64_MAX;
      if (pkey <= key) break;
      shard_of[b] = pw;
      --b;
    }
    shard_of[b] = w;
  }
  int rc = 0;
  for (uint64_t l = 0; l < n_layers; ++l) layer_shard[l] = UINT64_MAX;
  for (uint64_t s = 0; s < n_shards && rc == 0; ++s) {
    uint64_t w = shard_of[s];
    for (uint64_t i = 0; i < lens[w]; ++i) {
      uint64_t id = sets[w][i];
      if (layer_shard[id] != UINT64_MAX) {
        *bad_layer = id;
        *bad_shard_a = layer_shard[id];
        *bad_shard_b = s;
        rc = 1;
        break;
      }
      layer_shard[id] = s;
    }
  }
  if (rc == 0) {
    for (uint64_t l = 0; l < n_layers; ++l) {
      if (layer_shard[l] == UINT64_MAX) {
        *bad_layer = l;
        rc = 2;
        break;
      }
    }
  }
  if (rc == 0) {
    for (uint64_t s = 0; s < n_shards; ++s) shard_page_sizes[s] = 0;
    for (uint64_t l = 0; l < n_layers; ++l) {
      uint64_t s = layer_shard[l];
      layer_offsets[l] = shard_page_sizes[s];
      layer_bytes[l] = padded_bytes[l];
      shard_page_sizes[s] += padded_bytes[l];
    }
    *n_shards_out = n_shards;
  }
  for (uint64_t w = 0; w < n_sets; ++w) free(sets[w]);
  free(sets);
  free(lens);
  free(shard_of);
  return rc;
}

/* ----------------------------------------------------------------------- */
/* Whole-layer save / load over a host-resident cache, built from the       */
/* pieces above exactly as the reference composes them:                     */
/*   host image rule  offload.rs:454-509 (layer-first, batch allocation):   */
/*     split      -> K buffer and V buffer, block i at + i*padded_segment   */
/*     contiguous -> one buffer, block i at + i*padded_block                */
/*   descriptors      gpu_worker.rs:353-423                                 */
/*   copy             memcpy.rs / kernel.rs                                 */
/* `ids[i]` is the device slot of list position i.  host_k/host_v are the   */
/* two buffers (host_v unused when the layout is not split).                */
/* ----------------------------------------------------------------------- */

int orc_transfer_layer(const orc_layout* l, const uint32_t* ids, uint64_t n, uint8_t* host_k,
                       uint8_t* host_v, int host_is_src, int use_direct, int threads, char* err,
                       size_t cap) {
  if (n == 0) return ORC_OK;
  orc_desc* descs = (orc_desc*)malloc(sizeof(orc_desc) * n * 2);
  uint64_t m = 0;
  uint64_t stride = l->split ? l->padded_segment_bytes : l->padded_segment_bytes * l->segments;
  for (uint64_t i = 0; i < n; ++i) {
    uint64_t addr[2], bytes[2];
    int nc;
    if (orc_block_copies(l, ids[i], addr, bytes, &nc, err, cap)) {
      free(descs);
      return ORC_ERR;
    }
    uint64_t k = (uint64_t)(uintptr_t)host_k + i * stride;
    descs[m++] = (orc_desc){addr[0], k, k, bytes[0], 0, 1};
    if (nc == 2) {
      uint64_t v = (uint64_t)(uintptr_t)host_v + i * stride;
      descs[m++] = (orc_desc){addr[1], v, v, bytes[1], 0, 2};
    }
  }
  if (use_direct)
    orc_exec_direct(descs, m, host_is_src, threads);
  else
    orc_exec_kernel(descs, m, host_is_src, threads);
  free(descs);
  return ORC_OK;
}

/* Page-first variant (offload.rs:182-282): block i's page is pages[i]; this
 * layer's bytes sit at `offset` inside it. Split layouts are rejected by the
 * reference ("page-first save does not support split K/V"). */
int orc_transfer_layer_paged(const orc_layout* l, const uint32_t* ids, uint64_t n,
                             const uint64_t* pages, uint64_t offset, int host_is_src, int threads,
                             char* err, size_t cap) {
  if (l->split) return seterr(err, cap, "page-first save does not support split K/V");
  if (n == 0) return ORC_OK;
  orc_desc* descs = (orc_desc*)malloc(sizeof(orc_desc) * n);
  for (uint64_t i = 0; i < n; ++i) {
    uint64_t addr[2], bytes[2];
    int nc;
    if (orc_block_copies(l, ids[i], addr, bytes, &nc, err, cap)) {
      free(descs);
      return ORC_ERR;
    }
    uint64_t h = pages[i] + offset;
    descs[i] = (orc_desc){addr[0], h, h, bytes[0], 0, 100 + i};
  }
  orc_exec_kernel(descs, n, host_is_src, threads);
  free(descs);
  return ORC_OK;
}

size_t orc_sizeof_layout(void) { return sizeof(orc_layout); }
size_t orc_sizeof_desc(void) { return sizeof(orc_desc); }
size_t orc_sizeof_layer(void) { return sizeof(orc_layer); }
