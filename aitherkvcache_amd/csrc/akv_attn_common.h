// Work partition shared by the paged decode-attention kernels.
//
// The (sequence, KV block) pairs of a batch are laid end to end into one global block axis
// of length total = sum_i ceil(ctx_i / block_size).  The main kernel runs a fixed grid of G
// workgroups; workgroup w owns global blocks [w*per, (w+1)*per) with per = ceil(total / G),
// for ALL kv heads, and walks the sequences that range intersects.  Every (workgroup,
// sequence) intersection produces one partial (running max, running sum, unnormalised
// accumulator) per query head, stored in slot w + seq -- unique because both w and seq are
// non-decreasing along the walk and at least one of them grows at every step.  A reduce
// kernel merges the slots of a sequence with the log-sum-exp rule
// (aither_kvcache/fused_attention.py:513-522) and applies the inverse rotation.
// Everything is derived on the device from context_lens, so the launch needs no host
// synchronisation and the sequence can be recorded into a HIP graph.
#pragma once
#include "akv_common.h"

#define AKV_ATTN_WG_PER_CU 2

struct akv_attn_args {
  const uint8_t* kp; int64_t kps_blk, kps_pos, kps_head;
  const float* kn;   int64_t kns_blk, kns_pos, kns_head;
  const uint8_t* vp; int64_t vps_blk, vps_pos, vps_head;
  const float* vn;   int64_t vns_blk, vns_pos, vns_head;
  const void* block_tables; int bt_itype; int64_t bt_stride;
  const void* context_lens; int cl_itype;
  const float* centroids;
  int S, QH, KVH, block_size;
  int64_t max_blocks_per_seq;
  int64_t num_blocks;      // physical blocks in the cache; table entries are clamped into [0, num_blocks)
  float scale;
  const int32_t* prefix;
  const float* qrot;
  float* part_acc;
  float* part_ml;
  // matrix-core kernel only: a kv head with more than eight query heads is presented as `hgroup`
  // heads of QH / (KVH * hgroup) query heads each that read the same rows (KVH then counts those)
  int hgroup;
};

static inline int akv_attn_grid() {
  int cus = akv_cached_cu_count();
  return (cus > 0 ? cus : 256) * AKV_ATTN_WG_PER_CU;
}

static inline size_t akv_align256(size_t v) { return (v + 255) & ~(size_t)255; }

// Workspace carve-up.  acc_floats = floats of accumulator per query head
// (head_dim for the uniform codec, 256 for tq35).  The workspace starts with a header whose place
// does not depend on the batch: the cached lookup tables of the matrix-core kernels (their
// validity tag would otherwise outlive a call at another batch size that overwrote the words it
// vouches for) and the status words of the most recent call.
#define AKV_WS_LUT_BYTES 4096
#define AKV_WS_STATUS_BYTES 256
#define AKV_WS_HEADER_BYTES (AKV_WS_LUT_BYTES + AKV_WS_STATUS_BYTES)
// status word 0: nonzero when a bounded wait inside the main kernel of the most recent call gave up
// (cleared by the prologue, set with a plain vector store, turned into NaN outputs by the reduce)
#define AKV_STATUS_HANDOFF_TIMEOUT 1u
// record of a workgroup (int32 words): its range [g0, g1) of the global block axis; then its first segment: the
// sequence (-1: not recorded, the kernel searches the prefix), the sequence's first and one-past-last global
// block, its context length in tokens (clamped to the table width)
#define AKV_WGREC 8
#define AKV_WGREC_G0 0
#define AKV_WGREC_G1 1
#define AKV_WGREC_SEQ 2
#define AKV_WGREC_SB0 3
#define AKV_WGREC_SB1 4
#define AKV_WGREC_CTX 5
struct akv_attn_ws {
  uint32_t* lut;     // AKV_WS_LUT_BYTES of cached tables (matrix-core kernels)
  uint32_t* status;  // AKV_WS_STATUS_BYTES
  int32_t* wgdesc;   // [G][AKV_WGREC] record of every workgroup of the matrix-core kernel: its range of the global
                     // block axis and what its first segment starts from (written by that kernel's prologue; see
                     // akv_attn_partition)
  int32_t* seqw;     // [S][2] first and last workgroup whose range meets the sequence (same prologue)
  int32_t* prefix;   // [S + 1] exclusive prefix of blocks per sequence; prefix[S] = total
  float* qrot;       // [S][QH][acc_floats] transformed queries
  float* part_acc;   // [G + S][QH][acc_floats]
  float* part_ml;    // [G + S][QH][2]  (max, sum)
  size_t bytes;
};

static inline akv_attn_ws akv_attn_ws_layout(void* base, int S, int QH, int acc_floats, int G) {
  akv_attn_ws w;
  w.lut = (uint32_t*)base;
  w.status = (uint32_t*)((char*)base + AKV_WS_LUT_BYTES);
  size_t off = AKV_WS_HEADER_BYTES;
  w.wgdesc = (int32_t*)((char*)base + off);
  off += akv_align256((size_t)G * AKV_WGREC * 4);
  w.seqw = (int32_t*)((char*)base + off);
  off += akv_align256((size_t)(S > 0 ? S : 1) * 2 * 4);
  w.prefix = (int32_t*)((char*)base + off);
  off += akv_align256((size_t)(S + 1) * 4);
  w.qrot = (float*)((char*)base + off);
  off += akv_align256((size_t)S * QH * acc_floats * 4);
  w.part_acc = (float*)((char*)base + off);
  off += akv_align256((size_t)(G + S) * QH * acc_floats * 4);
  w.part_ml = (float*)((char*)base + off);
  off += akv_align256((size_t)(G + S) * QH * 2 * 4);
  w.bytes = off;
  return w;
}

// blocks a sequence occupies, clamped to the table width
__device__ __forceinline__ int akv_seq_blocks(const void* context_lens, int cl_itype, int s,
                                              int block_size, int64_t max_blocks_per_seq) {
  int64_t ctx = akv_load_index(context_lens, cl_itype, s);
  if (ctx < 0) ctx = 0;
  int64_t nb = (ctx + block_size - 1) / block_size;
  if (nb > max_blocks_per_seq) nb = max_blocks_per_seq;
  return (int)nb;
}

// physical block id of a table entry, clamped into the cache (a corrupt entry then reads a wrong
// block instead of memory outside the cache)
__device__ __forceinline__ int64_t akv_clamp_block(int64_t id, int64_t num_blocks) {
  return id < 0 ? 0 : (id >= num_blocks ? num_blocks - 1 : id);
}

__device__ __forceinline__ int64_t akv_seq_tokens(const void* context_lens, int cl_itype, int s,
                                                  int block_size, int64_t max_blocks_per_seq) {
  int64_t ctx = akv_load_index(context_lens, cl_itype, s);
  if (ctx < 0) ctx = 0;
  const int64_t cap = max_blocks_per_seq * block_size;
  return ctx < cap ? ctx : cap;
}

// One workgroup (256 threads) writes prefix[0..S].
__device__ __forceinline__ void akv_block_prefix_scan(const void* context_lens, int cl_itype, int S,
                                                      int block_size, int64_t max_blocks_per_seq,
                                                      int32_t* prefix, int32_t* scratch /*[>= 4] LDS*/) {
  const int tid = threadIdx.x;
  const int chunk = (S + 255) / 256;
  const int lo = min(S, tid * chunk), hi = min(S, lo + chunk);
  int sum = 0;
  for (int s = lo; s < hi; ++s) sum += akv_seq_blocks(context_lens, cl_itype, s, block_size, max_blocks_per_seq);
  // exclusive scan over the 256 threads: inclusive scan inside each wavefront by lane shifts, then
  // the four wavefront totals through LDS
  const int lane = tid & 63, wave = tid >> 6;
  const int inc = akv_wave_inclusive_scan(sum);
  if (lane == 63) scratch[wave] = inc;
  __syncthreads();
  int base = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int t = scratch[w];
    if (w < wave) base += t;
  }
  int run = base + inc - sum;
  for (int s = lo; s < hi; ++s) {
    prefix[s] = run;
    run += akv_seq_blocks(context_lens, cl_itype, s, block_size, max_blocks_per_seq);
  }
  if (tid == 255) prefix[S] = base + inc;
}

// ----------------------------------------------------------------------------------
// Block prefix of the batch and partition of the global block axis among the G workgroups of the matrix-core
// kernel, written by one workgroup of 256 threads.
//
// A workgroup whose range crosses a sequence boundary starts twice (query operand, block ids, first rows, a
// partial chunk at both ends): measured, such workgroups finish 5 us after the others and ARE the tail of
// the launch.  So when the batch has few sequences (at most 64 in all, the non-empty ones at most G / 8) every
// sequence gets whole workgroups: the smallest lambda (chunks per workgroup) with sum_s ceil(c_s / lambda) <= G
// is found by bisection (the sum is non-increasing in lambda), sequence s takes k_s = ceil(c_s / lambda)
// consecutive workgroups and splits its c_s chunks evenly among them; left-over workgroups get an empty range.
// Otherwise the axis is cut into G equal ranges as before.  Either way workgroups and sequences both advance
// monotonically along the axis, so slot = workgroup + sequence stays unique, and seqw[s] = (first, last
// workgroup that meets sequence s), which the reduce kernel reads instead of dividing by the range length.
// `cb` = blocks per chunk of the main kernel (2 for blocks of 16 tokens, 1 for blocks of 32).
// ----------------------------------------------------------------------------------
__device__ __forceinline__ void akv_attn_partition(int32_t* prefix, int S, int G, int cb, int32_t* wgdesc, int32_t* seqw,
                                                   int32_t* lds /*[>= 257]*/, const void* context_lens, int cl_itype,
                                                   int block_size, int64_t max_blocks_per_seq) {
  const int tid = threadIdx.x, lane = tid & 63;
  int32_t* p_wfirst = lds;              // [65] first workgroup of each sequence; [64] = workgroups in use
  int32_t* p_pref = lds + 65;           // [65] block prefix; [64] = total
  int32_t* p_ctx = lds + 130;           // [64] context length in tokens (clamped to the table width)
  int32_t* p_mode = lds + 194;          // [0] 1 = whole workgroups per sequence, [1] = total blocks
  if (S > 64) {
    // many sequences: the general scan, equal ranges, first segments found by the main kernel itself
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, lds);
    __threadfence_block();
    __syncthreads();                    // the prefix written by this workgroup is readable by all of it
    const int total = prefix[S];
    const int per = (total + G - 1) / G;
    for (int w = tid; w < G; w += blockDim.x) {
      int32_t* rec = wgdesc + (size_t)w * AKV_WGREC;
      const int g0 = min(total, w * per);
      rec[AKV_WGREC_G0] = g0;
      rec[AKV_WGREC_G1] = min(total, g0 + per);
      rec[AKV_WGREC_SEQ] = -1;
    }
    for (int s = tid; s < S; s += blockDim.x) {
      const int b0 = prefix[s], b1 = prefix[s + 1];
      const int w_lo = per > 0 ? b0 / per : 0;
      seqw[2 * s] = w_lo;
      seqw[2 * s + 1] = (per > 0 && b1 > b0) ? (b1 - 1) / per : w_lo - 1;
    }
    return;
  }
  // at most 64 sequences: one wavefront holds the batch, lane = sequence
  if (tid < 64) {
    int n = 0, ctx = 0;
    if (lane < S) {
      ctx = (int)akv_seq_tokens(context_lens, cl_itype, lane, block_size, max_blocks_per_seq);
      n = (ctx + block_size - 1) / block_size;
    }
    const int inc = akv_wave_inclusive_scan(n);
    const int total = __builtin_amdgcn_readlane(inc, 63);
    const int b0 = inc - n;
    if (lane < S) prefix[lane] = b0;
    if (lane == 0) prefix[S] = total;
    p_pref[lane] = b0;
    p_ctx[lane] = ctx;
    const int c = (n + cb - 1) / cb;                             // chunks of the lane's sequence
    const int sumc = akv_wave_sum(c);
    const int nz = __popcll(__ballot(c > 0));
    const int aligned = (nz >= 1 && nz * 8 <= G) ? 1 : 0;
    if (aligned) {
      int lo = (sumc + G - 1) / G, hi = (sumc + (G - nz) - 1) / (G - nz);      // hi is always feasible
      if (lo < 1) lo = 1;
      while (lo < hi) {
        const int mid = (lo + hi) >> 1;
        const int tot = akv_wave_sum((c + mid - 1) / mid);
        if (tot <= G) hi = mid; else lo = mid + 1;
      }
      const int k = (c + lo - 1) / lo;
      const int kinc = akv_wave_inclusive_scan(k);
      p_wfirst[lane] = kinc - k;
      if (lane == 63) p_wfirst[64] = kinc;
      if (lane < S) {
        seqw[2 * lane] = kinc - k;
        seqw[2 * lane + 1] = kinc - 1;
      }
    } else if (lane < S) {
      const int per = (total + G - 1) / G;
      const int w_lo = per > 0 ? b0 / per : 0;
      seqw[2 * lane] = w_lo;
      seqw[2 * lane + 1] = (per > 0 && n > 0) ? (b0 + n - 1) / per : w_lo - 1;
    }
    if (lane == 0) {
      p_pref[64] = total;
      p_mode[0] = aligned;
      p_mode[1] = total;
    }
  }
  __syncthreads();
  const int aligned = p_mode[0], total = p_mode[1];
  const int per = (total + G - 1) / G;
  for (int w = tid; w < G; w += blockDim.x) {
    int g0 = 0, g1 = 0, s = -1;
    if (aligned) {
      if (w < p_wfirst[64]) {
        // the last s with p_wfirst[s] <= w (entries are non-decreasing; a sequence without workgroups shares the
        // next one's entry and is passed over; entries of lanes past the batch equal the number in use)
        int cnt = 0;
        for (int i = 0; i < 64; ++i) cnt += (p_wfirst[i] <= w) ? 1 : 0;
        s = cnt - 1;
        const int b0 = p_pref[s], b1 = p_pref[s + 1];
        const int k = p_wfirst[s + 1] - p_wfirst[s];
        const int c = (b1 - b0 + cb - 1) / cb;
        const int pc = (c + k - 1) / k;
        g0 = min(b1, b0 + (w - p_wfirst[s]) * pc * cb);
        g1 = min(b1, g0 + pc * cb);
      }
    } else {
      g0 = min(total, w * per);
      g1 = min(total, g0 + per);
      if (g0 < g1) {
        int cnt = 0;
        for (int i = 0; i < 64; ++i) cnt += (i < S && p_pref[i] <= g0) ? 1 : 0;
        s = cnt - 1;      // the last sequence that starts at or before g0 (an empty one shares its successor's start)
      }
    }
    int32_t* rec = wgdesc + (size_t)w * AKV_WGREC;
    rec[AKV_WGREC_G0] = g0;
    rec[AKV_WGREC_G1] = g1;
    rec[AKV_WGREC_SEQ] = g0 < g1 ? s : -1;
    if (g0 < g1) {
      rec[AKV_WGREC_SB0] = p_pref[s];
      rec[AKV_WGREC_SB1] = p_pref[s + 1];
      rec[AKV_WGREC_CTX] = p_ctx[s];
    }
  }
}

// largest s with prefix[s] <= g  (prefix non-decreasing, prefix[0] = 0, g < prefix[S])
__device__ __forceinline__ int akv_find_seq(const int32_t* __restrict__ prefix, int S, int g) {
  int lo = 0, hi = S;  // invariant: prefix[lo] <= g < prefix[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (prefix[mid] <= g) lo = mid; else hi = mid;
  }
  return lo;
}

// The same search for a whole wavefront with up to 63 sequences: lane i holds prefix[i] (one vector load at the
// start of the kernel, `held`), the sequence is the number of entries 1..S that do not exceed g, and the bounds
// of the sequence come out of the register -- no chain of dependent loads per segment.  More sequences than
// that take the scalar search.
__device__ __forceinline__ int akv_prefix_hold(const int32_t* __restrict__ prefix, int S) {
  const int lane = threadIdx.x & 63;
  return prefix[min(lane, S)];
}
__device__ __forceinline__ int akv_find_seq_held(const int32_t* __restrict__ prefix, int S, int held, int g,
                                                 int& sb0, int& sb1) {
  if (S <= 63) {
    const int lane = threadIdx.x & 63;
    const int s = __popcll(__ballot(lane >= 1 && lane <= S && held <= g));
    sb0 = __builtin_amdgcn_readlane(held, s);
    sb1 = __builtin_amdgcn_readlane(held, s + 1);
    return s;
  }
  const int s = akv_find_seq(prefix, S, g);
  sb0 = prefix[s];
  sb1 = prefix[s + 1];
  return s;
}

// merge (m, l, acc) <- (m, l, acc) (+) (ms, ls, accs)
__device__ __forceinline__ void akv_lse_merge(float& m, float& l, float ms, float ls,
                                              float& alpha, float& beta) {
  const float mn = fmaxf(m, ms);
  if (mn == -INFINITY) { alpha = 1.f; beta = 0.f; return; }
  alpha = __expf(m - mn);
  beta = __expf(ms - mn);
  l = alpha * l + beta * ls;
  m = mn;
}

// ----------------------------------------------------------------------------------
// 128 x 128 rotations of a few float32 rows on the matrix cores (query rotation of the prologue,
// inverse rotation of the reduce).  The matrix comes as the float16 hi + lo operand tables of the
// prepared-rotation buffer (entries x 64; [hi | lo][8 N-tiles][4 k-steps][64 lanes] x 16 bytes, lane
// (col, g) = output coordinate 8 col + N-tile, contracted coordinates 32 g + 8 k-step + e).  A row is
// scaled by a power of two that brings its largest element to [1, 2) (exact), split into two float16
// terms rounded to nearest, and a tile is three products: hi.hi + hi.lo + lo.hi (~22 bits).
// ----------------------------------------------------------------------------------
typedef _Float16 akv_half8 __attribute__((ext_vector_type(8)));
typedef float akv_float4v __attribute__((ext_vector_type(4)));

// max over the four 16-lane rows of a wavefront, for every column (lane % 16)
__device__ __forceinline__ float akv_rows_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
// biased exponent used to scale a row whose largest magnitude is m (clamped so that both factors are normal)
__device__ __forceinline__ uint32_t akv_row_exponent(float m) {
  const uint32_t e = (__float_as_uint(m) >> 23) & 0xffu;
  return e < 1u ? 1u : (e > 253u ? 253u : e);
}
__device__ __forceinline__ float akv_row_scale(uint32_t e) { return __uint_as_float((254u - e) << 23); }     // 2^(127 - e)
__device__ __forceinline__ float akv_row_unscale(uint32_t e) { return __uint_as_float(e << 23); }             // 2^(e - 127)
// eight scaled values as two float16 operands
__device__ __forceinline__ void akv_split8(const float (&v)[8], float sc, akv_half8& hi, akv_half8& lo) {
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float x = v[e] * sc;
    const _Float16 h = (_Float16)x;
    hi[e] = h;
    lo[e] = (_Float16)(x - (float)h);
  }
}
__device__ __forceinline__ akv_half8 akv_as_half8(uint4 u) {
  union { uint4 u; akv_half8 h; } cv;
  cv.u = u;
  return cv.h;
}
// acc += (hi + lo) . (bh + bl) without the lo.lo term
__device__ __forceinline__ akv_float4v akv_mfma3(akv_half8 hi, akv_half8 lo, akv_half8 bh, akv_half8 bl, akv_float4v acc) {
  acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, bh, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi, bl, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo, bh, acc, 0, 0, 0);
  return acc;
}

