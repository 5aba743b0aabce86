// Streaming paged decode attention for the 4-bit cache in its dense layout
// ([blocks][block_size][8 kv heads][64 bytes] codes, [blocks][block_size][8] float32 norms),
// head_dim 128, block_size 16 or 32, at most 8 query heads per kv head.
//
// What the memory system sees is what a copy kernel would issue: every 16-token tile of K codes (8 KB
// contiguous), of V codes (8 KB) and the two 512-byte norm tiles are fetched exactly once, by loads in
// which the 64 lanes of a wavefront cover one contiguous kilobyte, and they go straight from the memory
// pipeline into LDS (global_load_lds_dwordx4: no registers, no LDS-write instructions).  The 16
// wavefronts of the workgroup share the fetching -- wavefront w of a role brings bytes [w KB, (w+1) KB)
// of each tile of its role's array -- and then each reads the rows of ITS kv head out of LDS:
//
//   wavefronts 0-7   SCORE role, kv head = wavefront: K codes -> scores on the matrix cores -> running
//                    softmax -> weights p * |v| handed over through LDS
//   wavefronts 8-15  VALUE role, same heads: V codes x weights on the matrix cores
//
// Chunks of 32 tokens (two tiles) flow through two rings of three slots (K and V).  A chunk passes two
// stages in a wavefront, one chunk period apart: the FRONT stage (during the work on chunk F) makes sure
// that chunk F + 1 is complete in LDS, copies the head's rows of it into registers and issues the loads of
// chunk F + 3 into the slot of chunk F; the BACK stage does the table lookups, products and softmax /
// accumulation on the rows copied a period earlier.  A trip through the LDS queue costs several hundred
// cycles when sixteen wavefronts keep it full; this way the trips the front stage needs overlap the lookups
// of the back stage instead of preceding them.
//
// Synchronisation is a handful of counters in LDS, one word per wavefront and kind, written without waiting
// (the LDS executes a wavefront's instructions in order) and polled once per chunk by ONE read in which
// lanes 0..7 look at `landed` of the own role (the wavefront's loads of the chunk are in LDS: it has executed
// a counted s_waitcnt vmcnt that covers them -- every issue step emits the same vector-memory instructions,
// real or repeated, so the count is a constant), lanes 8..15 at `copied` of the own role (rows taken into
// registers, the slot may be overwritten) and lane 16 at the partner wavefront of the head (`written`:
// weights of the chunk are in the exchange buffer; or the value side's `copied`, which it writes after
// taking the weights).  Every wait is bounded and a wait that gives up marks the call.
// A workgroup barrier per chunk needs no LDS instruction at all and was measured as well: it is 2 % slower
// and leaves no slack between wavefronts.
//
// What bounds the kernel (measured with cycle stamps and timing-only variants): not memory -- the counted
// waits for loads cost nothing, a variant without lookups and products streams 5.9 TB/s -- but the LDS
// pipe: it issues about one wavefront instruction every four to five cycles whatever its width, and the
// table lookups alone (one per code byte: 512 per chunk and workgroup) keep it 55 % busy at the speed
// reached, everything else (rows, norms, weights, counters) another 20 %.
//
// LDS map (160 KB): [0, 64 KB) table region, entry e at e * 256: 16 copies of (pair, remainder pair) in
// the first 128 bytes (a lookup is byte * 256 + (lane & 15) * 8: an 8-byte read serves 16 lanes per cycle,
// which then meet 16 different copies), the second 128 bytes are "fragment e", used for the weight
// exchange (20 fragments per head) and the norm tiles (one fragment per 4 tokens x 8 heads);
// [64 KB, 112 KB) K ring; [112 KB, 160 KB) V ring.
// Inside a K ring slot a tile keeps the cache's own order [token][head][64 bytes], except that the eight
// 16-byte pieces of every 128-byte line are stored at position (piece ^ (token & 7)): the loader lane
// that lands at position p fetches piece p ^ (token & 7) (its eight neighbours still cover the whole
// line), and lane (token n, quarter g) of a score wavefront reads its 16 bytes without bank conflicts.
// V tiles are stored as they are: lane (dword m, tokens 4g..4g+3) of a value wavefront reads its eight
// dwords with four two-address reads off one base register.
#include "akv_attn_common.h"
#include "akv_nibble.h"

typedef _Float16 sk_half8 __attribute__((ext_vector_type(8)));
typedef float sk_float4 __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const uint32_t sk_lds_cu32;
typedef __attribute__((address_space(3))) uint32_t sk_lds_u32;
typedef __attribute__((address_space(3))) sk_u32x4 sk_lds_u128;
typedef __attribute__((address_space(3))) void* sk_lds_ptr;
typedef __attribute__((address_space(1))) const void* sk_glb_ptr;

#define SK_THREADS 1024
#define SK_LDS_BYTES 163840
#define SK_KRING 65536u
#define SK_SLOT 16384u                       // one chunk of one array: two tiles of 16 tokens x 8 heads x 64 bytes
#define SK_TILE 8192u
#define SK_VRING (SK_KRING + 3u * SK_SLOT)
#define SK_FRAG(f) ((uint32_t)(f) * 256u + 128u)
#define SK_F_NORM 160                        // + ((slot * 2 + array) * 2 + tile) * 4 + token group
#define SK_F_CNT 208                         // counters: landed[role][8] (64 bytes) | copied[role][8] (64 bytes)
#define SK_F_CNT2 209                        // counters: weights written [8]
#define SK_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0f70 | (n))   // vmcnt(n), n < 16; other counters untouched
#define SK_W_VLO 256                         // words of the cached table block: remainder pairs, pairs, tag, marker, alpha
#define SK_W_VHI 512
#define SK_W_TAG 768
#define SK_W_MARK 784
#define SK_W_ALPHA 785
#define SK_MARK 0x9100u                     // differs from the marker of akv_attn_mfma.hip, whose block holds more tables
#define SK_ALPHA_CANDIDATES 65536

struct akv_stream_extra {
  const uint32_t* lut;
  const uint4* qop;       // [S][8 heads][8 k-steps][64 lanes] half8
  uint32_t* status;
  int spin_limit;
};

// ----------------------------------------------------------------------------------
// prologue: rotated queries in operand layout (scale * log2 e / alpha folded in before the hi / lo
// split), block prefix, lookup table
// ----------------------------------------------------------------------------------
// alpha in [1,2) minimising the largest relative fp16 rounding error of alpha * c over the levels;
// all 256 threads of the workgroup take part, every thread returns the result
__device__ __forceinline__ float sk_alpha_search(const float* __restrict__ centroids, int levels, float* best_err, float* best_alpha) {
  const int tid = threadIdx.x;
  float c[16];
  for (int v = 0; v < 16; ++v) c[v] = centroids[v & (levels - 1)];
  float berr = 1e30f, balpha = 1.f;
  for (int k = 0; k < SK_ALPHA_CANDIDATES / 256; ++k) {
    const float al = 1.f + (float)(tid * (SK_ALPHA_CANDIDATES / 256) + k) / (float)SK_ALPHA_CANDIDATES;
    float worst = 0.f;
    for (int v = 0; v < 16; ++v) {
      const float x = al * c[v];
      const float r = __half2float(__float2half_rn(x));
      const float e = x != 0.f ? fabsf(r - x) / fabsf(x) : 0.f;
      worst = fmaxf(worst, e);
    }
    if (worst < berr) { berr = worst; balpha = al; }
  }
  __syncthreads();
  best_err[tid] = berr;
  best_alpha[tid] = balpha;
  __syncthreads();
  if (tid == 0) {
    for (int t = 1; t < 256; ++t)
      if (best_err[t] < best_err[0]) { best_err[0] = best_err[t]; best_alpha[0] = best_alpha[t]; }
  }
  __syncthreads();
  return best_alpha[0];
}

template <int QDT>
__global__ __launch_bounds__(256) void akv_attn_stream_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ PiT,
    const float* __restrict__ centroids, int S, int QH, int KVH, const void* context_lens,
    int cl_itype, int block_size, int64_t max_blocks_per_seq, int32_t* prefix,
    uint4* __restrict__ qop, uint32_t* __restrict__ lut, uint32_t* __restrict__ status, int32_t* __restrict__ wgdesc,
    int G, float qscale, int bits) {
  __shared__ __align__(16) float q_lds[128][8];   // [input coordinate][query head of the group], zero-padded
  __shared__ float qr_lds[8][128];
  __shared__ int32_t scratch[257];
  __shared__ float best_err[256];
  __shared__ float best_alpha[256];
  __shared__ int stale;
  const int tid = threadIdx.x;
  const int nq = S * KVH;
  const int levels = 1 << bits;
  if ((int)blockIdx.x == nq) {
    if (tid == 0) status[0] = 0u;
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, scratch);
    // where every workgroup of the main kernel starts, so that it begins to fetch after one load:
    // range [g0, g1) of the global block axis, sequence and block of g0, blocks of the first segment, chunks
    __threadfence_block();
    __syncthreads();
    const int total = prefix[S];
    const int per = (total + G - 1) / G;
    for (int w = tid; w < G; w += 256) {
      const int64_t g0l = (int64_t)w * per;
      const int g0 = (int)(g0l < total ? g0l : total), g1 = min(total, g0 + per);
      int s0 = 0, blk0 = 0, nblk0 = 0, chunks = 0;
      if (g0 < g1) {
        s0 = akv_find_seq(prefix, S, g0);
        blk0 = g0 - prefix[s0];
        nblk0 = min(g1, prefix[s0 + 1]) - g0;
        int gcur = g0, s = s0;
        while (gcur < g1) {
          while (prefix[s + 1] <= gcur) ++s;
          const int nb = min(g1, prefix[s + 1]) - gcur;
          chunks += block_size == 32 ? nb : (nb + 1) >> 1;
          gcur += nb;
        }
      }
      int32_t* d = wgdesc + (size_t)w * 8;
      d[0] = g0; d[1] = g1; d[2] = s0; d[3] = blk0; d[4] = nblk0; d[5] = chunks; d[6] = 0; d[7] = 0;
    }
    return;
  }
  // the cached table block is valid when its marker and the centroids it was built from match
  if (tid == 0) stale = (lut[SK_W_MARK] != SK_MARK + (uint32_t)bits) ? 1 : 0;
  __syncthreads();
  if (tid < levels && __float_as_uint(centroids[tid]) != lut[SK_W_TAG + tid]) stale = 1;
  __syncthreads();
  const bool is_stale = stale != 0;
  if ((int)blockIdx.x == nq + 1) {
    if (!is_stale) return;
    const float al = sk_alpha_search(centroids, levels, best_err, best_alpha);
    if (tid == 0) lut[SK_W_ALPHA] = __float_as_uint(al);
    const float c0 = centroids[(tid >> 4) & (levels - 1)], c1 = centroids[tid & 15 & (levels - 1)];
    const __half v0 = __float2half_rn(al * c0), v1 = __float2half_rn(al * c1);
    lut[SK_W_VHI + tid] = (unsigned)__half_as_ushort(v0) | ((unsigned)__half_as_ushort(v1) << 16);
    const __half l0 = __float2half_rn(al * c0 - __half2float(v0)), l1 = __float2half_rn(al * c1 - __half2float(v1));
    lut[SK_W_VLO + tid] = (unsigned)__half_as_ushort(l0) | ((unsigned)__half_as_ushort(l1) << 16);
    if (tid < levels) lut[SK_W_TAG + tid] = __float_as_uint(centroids[tid]);
    __threadfence();
    __syncthreads();
    if (tid == 0) lut[SK_W_MARK] = SK_MARK + (uint32_t)bits;
    return;
  }
  // a workgroup that finds the block stale derives alpha itself (the same search, the same result) instead
  // of waiting for the workgroup that rebuilds the block
  const float alpha = is_stale ? sk_alpha_search(centroids, levels, best_err, best_alpha) : __uint_as_float(lut[SK_W_ALPHA]);
  const float qs_eff = qscale / alpha;
  const int s = blockIdx.x / KVH, h = blockIdx.x % KVH;
  const int gqa = QH / KVH;
  const int dim = tid & 127, half = tid >> 7;
  float pvr[64];
#pragma unroll
  for (int jj = 0; jj < 64; ++jj) pvr[jj] = PiT[(half * 64 + jj) * 128 + dim];
  for (int i = tid; i < 8 * 128; i += 256) {
    const int q = i >> 7, j = i & 127;
    q_lds[j][q] = q < gqa ? akv_elem<QDT>::load(query, s * qs_seq + (h * gqa + q) * qs_head + j) : 0.f;
  }
  __syncthreads();
  {
    float part[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) part[q] = 0.f;
#pragma unroll
    for (int jj = 0; jj < 64; ++jj) {
      const int j = half * 64 + jj;
      const float pv = pvr[jj];
      const float4 qa = *(const float4*)&q_lds[j][0];
      const float4 qc = *(const float4*)&q_lds[j][4];
      part[0] = fmaf(pv, qa.x, part[0]); part[1] = fmaf(pv, qa.y, part[1]);
      part[2] = fmaf(pv, qa.z, part[2]); part[3] = fmaf(pv, qa.w, part[3]);
      part[4] = fmaf(pv, qc.x, part[4]); part[5] = fmaf(pv, qc.y, part[5]);
      part[6] = fmaf(pv, qc.z, part[6]); part[7] = fmaf(pv, qc.w, part[7]);
    }
    if (half == 1) {
#pragma unroll
      for (int q = 0; q < 8; ++q) qr_lds[q][dim] = part[q];
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int q = 0; q < 8; ++q) qr_lds[q][dim] = (qr_lds[q][dim] + part[q]) * qs_eff;
    }
  }
  __syncthreads();
  // operand of k-step n (dword n / 2 of the lane's four, bytes 2 (n % 2) and 2 (n % 2) + 1): lane (col, g),
  // element e faces byte 2 (n % 2) + e / 4, nibble e % 2; elements 2,3 and 6,7 repeat 0,1 and 4,5 (they face
  // the remainder halves of the table entries); columns [0,8) hold the fp16 rounding of q', columns [8,16)
  // the fp16 of the remainder
  for (int n = tid >> 6; n < 8; n += 4) {
    const int lane = tid & 63;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int st = n >> 1, b = 2 * (n & 1) + (e >> 2), lo = e & 1;
      const int d = 32 * g + (bits == 4 ? mf_kcoord<4>(st, b, lo) : bits == 3 ? mf_kcoord<3>(st, b, lo) : mf_kcoord<2>(st, b, lo));
      float v = 0.f;
      if (col < 8) {
        if (col < gqa) v = __half2float(__float2half_rn(qr_lds[col][d]));
      } else if (col - 8 < gqa) {
        const float full = qr_lds[col - 8][d];
        v = full - __half2float(__float2half_rn(full));
      }
      hbits[e] = __half_as_ushort(__float2half_rn(v));
    }
    uint4 o;
    o.x = hbits[0] | (hbits[1] << 16); o.y = hbits[2] | (hbits[3] << 16);
    o.z = hbits[4] | (hbits[5] << 16); o.w = hbits[6] | (hbits[7] << 16);
    qop[((size_t)(s * KVH + h) * 8 + n) * 64 + lane] = o;
  }
}

// ----------------------------------------------------------------------------------
// main kernel helpers
// ----------------------------------------------------------------------------------
typedef uint32_t sk_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const sk_u32x2 sk_lds_cu64;
#define SK_SEL(k) (0x0c020400u + ((uint32_t)(k) << 8))
// table lookups: address = byte k of `word` * 256 + lanebits, one byte permute
__device__ __forceinline__ sk_u32x2 sk_lut2(uint32_t lanebits, uint32_t word, uint32_t sel) {   // (pair, remainder pair)
  const uint32_t addr = __builtin_amdgcn_perm(word, lanebits, sel);
  return *(sk_lds_cu64*)(uintptr_t)addr;
}
__device__ __forceinline__ uint32_t sk_lut(uint32_t lanebits, uint32_t word, uint32_t sel) {      // pair
  const uint32_t addr = __builtin_amdgcn_perm(word, lanebits, sel);
  return *(sk_lds_cu32*)(uintptr_t)addr;
}
__device__ __forceinline__ sk_half8 sk_pack(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  union { uint32_t u[4]; sk_half8 h; } x;
  x.u[0] = a; x.u[1] = b; x.u[2] = c; x.u[3] = d;
  return x.h;
}
__device__ __forceinline__ float sk_from_hi_cols(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x108 /*row_shl:8*/, 0xf, 0xf, true));
}
__device__ __forceinline__ float sk_from_lo_cols(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x118 /*row_shr:8*/, 0xf, 0xf, true));
}
// value of lane N of the own row of 16 lanes
template <int N>
__device__ __forceinline__ float sk_row_bcast(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x150 + N /*row_newbcast:N*/, 0xf, 0xf, true));
}
__device__ __forceinline__ uint64_t sk_umul(uint32_t a, uint32_t b) { return (uint64_t)a * (uint64_t)b; }
__device__ __forceinline__ uint32_t sk_here(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}
__device__ __forceinline__ float sk_rows_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float sk_rows_sum(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// 16 bytes per lane from global memory straight into LDS at lds_dst + lane * 16 (lds_dst wavefront-uniform)
__device__ __forceinline__ void sk_dma16(const void* src, uint32_t lds_dst) {
  __builtin_amdgcn_global_load_lds((sk_glb_ptr)src, (sk_lds_ptr)(uintptr_t)lds_dst, 16, 0, 0);
}
// Progress counters.  LDS operations of a wavefront execute in order, so a counter written after data is seen
// after the data, and a counter written after reads is written after they have fetched their data.  The wait
// polls one LDS word per lane (which word, and the threshold `need` it must reach, are the lane's own; 0 for
// the lanes that watch nothing).  It is bounded: a wait that gives
// up marks the call (an ordinary vector store), the kernel goes on with whatever LDS holds, the reduce kernel
// turns every output of the call into NaN and akv_paged_attn_status reports it.
__device__ __forceinline__ void sk_publish(uint32_t addr, uint32_t value) {
  asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");     // no wait: the LDS keeps a wavefront's order
}
__device__ __forceinline__ void sk_give_up(uint32_t* status) {
  if ((threadIdx.x & 63) == 0) *(volatile uint32_t*)status = AKV_STATUS_HANDOFF_TIMEOUT;
}
__device__ __forceinline__ void sk_wait_progress(uint32_t addr, uint32_t need, uint32_t* status, int limit) {
  for (int spin = 0; spin < limit; ++spin) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    if (__builtin_amdgcn_ballot_w64((int32_t)(v - need) < 0) == 0) return;
    __builtin_amdgcn_s_sleep(2);
  }
  if ((threadIdx.x & 63) == 0) *(volatile uint32_t*)status = AKV_STATUS_HANDOFF_TIMEOUT;
}

// The workgroup's share of the global block axis as a walk over segments (the intersections of its
// range with the sequences).  Scalar state only.
struct sk_walk {
  int gcur;          // first global block not yet walked
  int s;             // sequence of the current segment
  int blk_lo, nblk;  // its blocks inside the sequence
  int nchunks;
  bool valid;
};

// ----------------------------------------------------------------------------------
// main kernel
// ----------------------------------------------------------------------------------
template <int ROLE>
__device__ __forceinline__ void sk_role_main(const akv_attn_args& a, const akv_stream_extra& x,
                                             const int32_t* __restrict__ prefix, const void* __restrict__ block_tables,
                                             const void* __restrict__ context_lens, const int32_t* __restrict__ wgdesc,
                                             const int hs) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const uint32_t lanebits = (uint32_t)(lane & 15) * 8u;
  // exchange of head slot hs: weights (16 bytes per lane) in fragments 20 hs + 8 par + lane / 8, rescale factors
  // (4 bytes per lane) in fragments 20 hs + 16 + 2 par + lane / 32; parity 1 lies a constant further on
  const uint32_t pb_addr = SK_FRAG(20 * hs + (lane >> 3)) + (uint32_t)(lane & 7) * 16u;
  const uint32_t rs_addr = SK_FRAG(20 * hs + 16 + (lane >> 5)) + (uint32_t)(lane & 31) * 4u;
  constexpr uint32_t PB_PAR = 8u * 256u, RS_PAR = 2u * 256u;

  const bool bs32 = a.block_size == 32;
  const int bs = bs32 ? 32 : 16;
  // where this workgroup starts: one 32-byte record written by the prologue (no search, no chain of loads
  // before the first fetch goes out)
  const int32_t* const desc = wgdesc + (size_t)blockIdx.x * 8;
  const int g0 = desc[0], g1 = desc[1];
  const uint32_t N = (uint32_t)desc[5];       // chunks of the whole range
  const int gqa = a.QH / a.KVH;
  const bool idle = g0 >= g1;                 // no blocks for this workgroup (it still takes part in the table fill)
  uint32_t* const status = x.status;
  const int limit = x.spin_limit;
  // Counters, one word per wavefront and kind, each the number of chunks the wavefront has taken that far:
  //   landed  its own loads of the chunk are in LDS (it has executed a counted wait that covers them)
  //   copied  it has copied its head's rows of the chunk (and, value role, the weights) into registers
  //   written (score role) the weights of the chunk are in the exchange buffer
  // The lane's word in a poll: lanes 0..7 `landed` of the own role, lanes 8..15 `copied` of the own role,
  // lane 16 the partner's (`copied` of the value wavefront for a score wavefront -- in a round it is written
  // after the weights were taken --, `written` for a value one).
  const uint32_t cnt_landed = SK_FRAG(SK_F_CNT) + 32u * ROLE + 4u * (uint32_t)hs;
  const uint32_t cnt_copied = SK_FRAG(SK_F_CNT) + 64u + 32u * ROLE + 4u * (uint32_t)hs;
  const uint32_t cnt_written = SK_FRAG(SK_F_CNT2) + 4u * (uint32_t)hs;
  const uint32_t cnt_partner = ROLE == 0 ? SK_FRAG(SK_F_CNT) + 64u + 32u + 4u * (uint32_t)hs : cnt_written;
  const uint32_t cnt_poll = lane < 16 ? SK_FRAG(SK_F_CNT) + 32u * ROLE + (lane < 8 ? 0u : 64u) + 4u * (uint32_t)(lane & 7)
                                      : (lane == 16 ? cnt_partner : SK_FRAG(SK_F_CNT));

  // ---- walk over the segments of [g0, g1): the first comes from the record, later ones are the next
  // sequences that own blocks
  auto walk_first = [&](sk_walk& w) {
    w.s = desc[2]; w.blk_lo = desc[3]; w.nblk = desc[4];
    w.nchunks = bs32 ? w.nblk : (w.nblk + 1) >> 1;
    w.gcur = g0 + w.nblk;
    w.valid = !idle;
  };
  auto walk_begin = [&](sk_walk& w) {
    if (w.gcur >= g1) { w.valid = false; return; }
    int s = w.s + 1;
    while (prefix[s + 1] <= w.gcur) ++s;      // sequences without blocks; stops before a.S because gcur < total
    w.s = s;
    const int sb0 = prefix[s], sb1 = prefix[s + 1];
    w.blk_lo = w.gcur - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    w.nblk = blk_hi - w.blk_lo;
    w.nchunks = bs32 ? w.nblk : (w.nblk + 1) >> 1;
    w.gcur = sb0 + blk_hi;
    w.valid = true;
  };

  // ---- the loading side: one issue step per chunk, in walk order, always the same vector-memory
  // instructions (score role 4, value role 2); past the end of the range it re-reads block 0 into the
  // slot whose turn it is (free by then), so that the instruction counts behind the waits never change
  sk_walk lw;
  walk_first(lw);
  int lc = 0;                 // chunk of the loader's segment
  uint32_t l_slot = 0;        // ring slot of the next issue step
  const unsigned char* const codes = ROLE == 0 ? a.kp : a.vp;
  const uint32_t cps_blk = (uint32_t)(ROLE == 0 ? a.kps_blk : a.vps_blk);
  const uint32_t ring = ROLE == 0 ? SK_KRING : SK_VRING;
  // K loader lane -> (token 2 hs + lane / 32, 128-byte line (lane / 8) % 4, position lane % 8 holding piece
  // position ^ (token & 7)); V loader lane -> its 16 bytes of the wavefront's kilobyte
  const uint32_t ld_tok = 2u * (uint32_t)hs + (uint32_t)(lane >> 5);
  const uint32_t ld_voff = ROLE == 0 ? ld_tok * 512u + (uint32_t)((lane >> 3) & 3) * 128u + (((uint32_t)lane & 7u) ^ (ld_tok & 7u)) * 16u
                                     : (uint32_t)hs * 1024u + (uint32_t)lane * 16u;
  const uint32_t tile1_off = bs32 ? 16u * 512u : 0u;
  // norm tiles (score role): wavefront hs brings tokens 4 (hs % 4) .. + 3 of tile hs / 4, lanes 0..7
  const int nj = hs >> 2, nq = hs & 3;
  const uint32_t nrm_voff = (uint32_t)nq * 32u + (uint32_t)(lane & 7) * 4u;      // floats
  const uint32_t nrm_tile1 = bs32 ? 128u : 0u;
  auto issue = [&]() {
    uint32_t p0 = 0, p1 = 0;
    if (lw.valid) {
      const int bi = lw.blk_lo + (bs32 ? lc : 2 * lc);
      const int64_t row = (int64_t)lw.s * a.bt_stride + bi;
      p0 = (uint32_t)akv_clamp_block(akv_load_index(block_tables, a.bt_itype, row), a.num_blocks);
      p1 = p0;
      if (!bs32 && 2 * lc + 1 < lw.nblk)
        p1 = (uint32_t)akv_clamp_block(akv_load_index(block_tables, a.bt_itype, row + 1), a.num_blocks);
      if (++lc == lw.nchunks) { lc = 0; walk_begin(lw); }
    }
    const uint32_t dst = ring + l_slot * SK_SLOT + (uint32_t)hs * 1024u;
    sk_dma16(codes + sk_umul(p0, cps_blk) + sk_here(ld_voff), dst);
    sk_dma16(codes + sk_umul(p1, cps_blk) + tile1_off + sk_here(ld_voff), dst + SK_TILE);
    if constexpr (ROLE == 0) {
      const uint32_t pj = nj ? p1 : p0;
      const uint32_t noff = nj ? nrm_tile1 : 0u;
      const uint32_t fk = SK_FRAG(SK_F_NORM + ((l_slot * 2 + 0) * 2 + nj) * 4 + nq);
      const uint32_t fv = SK_FRAG(SK_F_NORM + ((l_slot * 2 + 1) * 2 + nj) * 4 + nq);
      if (lane < 8) {
        sk_dma16(a.kn + sk_umul(pj, (uint32_t)a.kns_blk) + noff + sk_here(nrm_voff), fk);
        sk_dma16(a.vn + sk_umul(pj, (uint32_t)a.vns_blk) + noff + sk_here(nrm_voff), fv);
      }
    }
    l_slot = l_slot == 2 ? 0 : l_slot + 1;
  };

  // ---- the first two chunks are requested before anything else; while they travel, the lookup table is
  // written (all wavefronts of the workgroup, one barrier)
  sk_walk cw;
  walk_first(cw);
  // the segment being consumed (cw always describes the one after it)
  int s = cw.s, nchunks = cw.nchunks, nblk = cw.nblk, blk_lo = cw.blk_lo;
  int c = 0;
  // The query operand lives in 32 registers for a whole segment and is replaced in place at a segment's
  // last chunk.  The loads are written as assembly so that the compiler keeps no score of them (it would
  // wait for ALL outstanding loads, prefetched chunks included, before the first product of every chunk);
  // the counted wait at the top of the next chunk covers them: they are older than the chunk loads issued
  // behind them.  "+v" keeps each operand in the registers it already has.
  sk_half8 qb[8];
#pragma unroll
  for (int st = 0; st < 8; ++st) qb[st] = (sk_half8){0, 0, 0, 0, 0, 0, 0, 0};
  auto load_q = [&](int seq) {
    const uint4* qp = x.qop + ((size_t)(seq * a.KVH + hs) * 8) * 64 + lane;
    const uint4* qp2 = qp + 4 * 64;
    asm volatile("global_load_dwordx4 %0, %4, off\n\t"
                 "global_load_dwordx4 %1, %4, off offset:1024\n\t"
                 "global_load_dwordx4 %2, %4, off offset:2048\n\t"
                 "global_load_dwordx4 %3, %4, off offset:3072"
                 : "+v"(qb[0]), "+v"(qb[1]), "+v"(qb[2]), "+v"(qb[3]) : "v"(qp) : "memory");
    asm volatile("global_load_dwordx4 %0, %4, off\n\t"
                 "global_load_dwordx4 %1, %4, off offset:1024\n\t"
                 "global_load_dwordx4 %2, %4, off offset:2048\n\t"
                 "global_load_dwordx4 %3, %4, off offset:3072"
                 : "+v"(qb[4]), "+v"(qb[5]), "+v"(qb[6]), "+v"(qb[7]) : "v"(qp2) : "memory");
  };
  // the thread's share of the lookup table (and alpha) is requested first, so that the wait before the
  // table is written leaves the chunk loads behind it in flight
  const int tb_e = threadIdx.x >> 2, tb_q = threadIdx.x & 3;
  const uint32_t tb_hi = x.lut[SK_W_VHI + tb_e], tb_lo = x.lut[SK_W_VLO + tb_e];
  const float alpha = __uint_as_float(x.lut[SK_W_ALPHA]);
  __builtin_amdgcn_sched_barrier(0);
  issue();          // (a workgroup without blocks reads block 0 like any wavefront past the end of its range)
  __builtin_amdgcn_sched_barrier(0);
  issue();
  __builtin_amdgcn_sched_barrier(0);
  issue();          // the three slots of the ring are all free at the start
  __builtin_amdgcn_sched_barrier(0);
  SK_WAIT_VM(0);    // the table words and the three chunks have landed (the table is needed before any of them is used)
  {
    // entry e at e * 256: 16 copies of (pair, remainder pair); thread (e, quarter) writes four of them
    // (written as assembly: the compiler would hold these LDS stores back until the chunk loads, which also
    // write LDS, have all landed)
    const uint32_t va = (uint32_t)tb_e * 256u + (uint32_t)tb_q * 32u;
    const sk_u32x4 word = (sk_u32x4){tb_hi, tb_lo, tb_hi, tb_lo};
    asm volatile("ds_write_b128 %0, %1\n\tds_write_b128 %0, %1 offset:16" : : "v"(va), "v"(word) : "memory");
    if (threadIdx.x < 64) {
      const uint32_t ca = (threadIdx.x < 32 ? SK_FRAG(SK_F_CNT) : SK_FRAG(SK_F_CNT2) - 128u) + 4u * threadIdx.x, zero = 0u;
      asm volatile("ds_write_b32 %0, %1" : : "v"(ca), "v"(zero) : "memory");
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  }
  const float inv_alpha = 1.f / alpha;
  asm volatile("" : : "v"(inv_alpha));      // alpha has arrived with the table words: no wait for it inside the loop
  __syncthreads();
  if (idle) {
    SK_WAIT_VM(0);
    return;
  }
  if constexpr (ROLE == 0) load_q(s);       // behind the chunk loads in the queue: the first wait of the loop covers them
  __builtin_amdgcn_sched_barrier(0);
  walk_begin(cw);

  // Every chunk goes through two stages in a wavefront, one chunk period apart:
  //   front  (during the work on chunk F): make sure chunk F + 1 is complete in LDS, copy the head's rows of it
  //          into registers, issue the loads of chunk F + 3 into the slot of chunk F (which everybody copied a
  //          period ago)
  //   back   table lookups, products, softmax / accumulation on the rows copied a period earlier
  // so that the trips through the LDS queue that the front stage needs (counters, rows: several hundred
  // cycles each when sixteen wavefronts keep the queue full) overlap the lookups of the back stage instead of
  // preceding them.
  if constexpr (ROLE == 0) {
    // =========================== score wavefront ===========================
    // reader: lane (token col, quarter g) -> 16 bytes of row (col, hs)
    const uint32_t kaddr = SK_KRING + (uint32_t)col * 512u + (uint32_t)(hs >> 1) * 128u +
                           ((((uint32_t)(hs & 1) * 4u + (uint32_t)g) ^ ((uint32_t)col & 7u)) * 16u);
    // one norm per lane: lane (col, g) -> array col / 8 (K | V), tile (col / 4) % 2, token 4 g + col % 4;
    // fragment (slot, array, tile, g), float [token][head]
    const uint32_t naddr = SK_FRAG(SK_F_NORM + ((col >> 3) * 2 + ((col >> 2) & 1)) * 4 + g) + (uint32_t)(col & 3) * 32u + (uint32_t)hs * 4u;
    float m_run = -INFINITY, l_run = 0.f;
    int64_t ctx = akv_seq_tokens(context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
    int t_end = (int)min((int64_t)(blk_lo + nblk) * bs, ctx);

    // chunks 0..2 have landed (waited for before the table was written); copy chunk 0
    sk_publish(cnt_landed, 3u);
    sk_wait_progress(cnt_poll, lane < 8 ? 1u : 0u, status, limit);
    sk_u32x4 kc0 = *(sk_lds_u128*)(uintptr_t)(kaddr);
    sk_u32x4 kc1 = *(sk_lds_u128*)(uintptr_t)(kaddr + SK_TILE);
    float nv = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(naddr));
    sk_publish(cnt_copied, 1u);
    uint32_t r_slot = 1;          // slot of the chunk the front stage copies next

    for (uint32_t F = 0; F < N; ++F) {
      const bool last = c == nchunks - 1;
      const bool more = F + 1u < N;
      const uint32_t kw[8] = {kc0.x, kc0.y, kc0.z, kc0.w, kc1.x, kc1.y, kc1.z, kc1.w};
      const float nv_cur = nv;
      sk_u32x2 w[5][4];      // ring of five dwords of lookups: four in flight behind the one multiplied
      sk_float4 acc[2];
      acc[0] = (sk_float4){0.f, 0.f, 0.f, 0.f};
      acc[1] = (sk_float4){0.f, 0.f, 0.f, 0.f};
      // ---- back stage, first lookups of chunk F
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int b = 0; b < 4; ++b) w[n][b] = sk_lut2(lanebits, kw[n], SK_SEL(b));
      __builtin_amdgcn_sched_barrier(0);
      // ---- front stage.  Chunk F + 1 is complete in LDS (every score wavefront has said so), everybody has
      // copied chunk F out of the slot that the loads of chunk F + 3 are about to overwrite, and the value
      // wavefront of this head has taken the weights of chunk F - 2, whose buffer this chunk's will go into
      // (its `copied` counter reached F in the round in which it took them).
      // (the second condition holds for the re-reads of block 0 past the end of the range as well: they land in
      // the ring like any chunk)
      sk_wait_progress(cnt_poll, lane < 8 ? (more ? F + 2u : 0u) : (lane < 16 ? F + 1u : (lane == 16 && F >= 2u ? F : 0u)), status, limit);
      if (more) {
        const uint32_t slot_off = r_slot * SK_SLOT;
        kc0 = *(sk_lds_u128*)(uintptr_t)(kaddr + slot_off);
        kc1 = *(sk_lds_u128*)(uintptr_t)(kaddr + slot_off + SK_TILE);
        nv = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(naddr + r_slot * 16u * 256u));
        r_slot = r_slot == 2 ? 0 : r_slot + 1;
        asm volatile("" ::: "memory");
        sk_publish(cnt_copied, F + 2u);       // queued behind the reads: executed once they have fetched their data
      }
      __builtin_amdgcn_sched_barrier(0);
      if (!last) issue();             // chunk F + 3 into the slot of chunk F
      __builtin_amdgcn_sched_barrier(0);
      // first chunk of a segment: the queries requested at the end of the previous one (or at the start of the
      // kernel) are needed now; the only loads issued behind them are those of one chunk
      if (c == 0) {
        if (F == 0u && last) SK_WAIT_VM(0); else SK_WAIT_VM(4);
      }
      __builtin_amdgcn_sched_barrier(0);
      // ---- back stage: 16 k-steps (tile j, dword st, byte pair), two table reads (each a pair and its remainder) feed one MFMA
#pragma unroll
      for (int n = 0; n < 8; ++n) {
        if (n + 4 < 8) {
#pragma unroll
          for (int b = 0; b < 4; ++b) w[(n + 4) % 5][b] = sk_lut2(lanebits, kw[n + 4], SK_SEL(b));
        }
        acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            sk_pack(w[n % 5][0].x, w[n % 5][0].y, w[n % 5][1].x, w[n % 5][1].y), qb[2 * (n & 3)], acc[n >> 2], 0, 0, 0);
        acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            sk_pack(w[n % 5][2].x, w[n % 5][2].y, w[n % 5][3].x, w[n % 5][3].y), qb[2 * (n & 3) + 1], acc[n >> 2], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (last) {
        // this wavefront's loads of chunk F + 2 have landed (nothing newer is in the queue yet)
        SK_WAIT_VM(0);
        sk_publish(cnt_landed, F + 3u);
        __builtin_amdgcn_sched_barrier(0);
        // the queries of the next segment take the place of this one's now that its last product is issued (the
        // counted wait of the next chunk covers them: they are older than the chunk loads issued behind them)
        if (cw.valid) load_q(cw.s);
        __builtin_amdgcn_sched_barrier(0);
        issue();
      } else {
        // this wavefront's loads of chunk F + 2 have landed (4 newer instructions, those of chunk F + 3; chunk
        // F + 2 was requested a chunk period ago, so this seldom waits)
        SK_WAIT_VM(4);
        sk_publish(cnt_landed, F + 3u);
      }
      __builtin_amdgcn_sched_barrier(0);
      float sv[8];
      // columns c and c + 8 carry the hi and lo part of the same query head; K norms come from the lanes that hold them
      sv[0] = (acc[0][0] + sk_from_hi_cols(acc[0][0])) * sk_row_bcast<0>(nv_cur);
      sv[1] = (acc[0][1] + sk_from_hi_cols(acc[0][1])) * sk_row_bcast<1>(nv_cur);
      sv[2] = (acc[0][2] + sk_from_hi_cols(acc[0][2])) * sk_row_bcast<2>(nv_cur);
      sv[3] = (acc[0][3] + sk_from_hi_cols(acc[0][3])) * sk_row_bcast<3>(nv_cur);
      sv[4] = (acc[1][0] + sk_from_hi_cols(acc[1][0])) * sk_row_bcast<4>(nv_cur);
      sv[5] = (acc[1][1] + sk_from_hi_cols(acc[1][1])) * sk_row_bcast<5>(nv_cur);
      sv[6] = (acc[1][2] + sk_from_hi_cols(acc[1][2])) * sk_row_bcast<6>(nv_cur);
      sv[7] = (acc[1][3] + sk_from_hi_cols(acc[1][3])) * sk_row_bcast<7>(nv_cur);
      uint32_t dead = 0;            // bit 4 j + i: token 4 g + i of tile j lies outside the context
      if (last) {                   // only the last chunk of a segment can hold masked tokens
        const int tok0 = blk_lo * bs + 32 * c;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int tok = tok0 + 16 * j + 4 * g + i;
            const bool ok = (tok < t_end) && (j == 0 || bs32 || 2 * c + 1 < nblk);
            if (!ok) { sv[4 * j + i] = -INFINITY; dead |= 1u << (4 * j + i); }
          }
      }
      // running softmax in the log2 domain (scale * log2 e is folded into the query operand)
      float mx = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])), fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
      mx = sk_rows_max(mx);
      const float m_new = fmaxf(m_run, mx);
      const float resc = __builtin_amdgcn_exp2f(m_run - m_new);   // 0 on the first chunk
      m_run = m_new;
      float psum = 0.f;
      float pw[8];
      {
        float p[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          p[i] = __builtin_amdgcn_exp2f(sv[i] - m_new);    // 0 for masked tokens
          psum += p[i];
        }
        pw[0] = p[0] * sk_row_bcast<8>(nv_cur);  pw[1] = p[1] * sk_row_bcast<9>(nv_cur);
        pw[2] = p[2] * sk_row_bcast<10>(nv_cur); pw[3] = p[3] * sk_row_bcast<11>(nv_cur);
        pw[4] = p[4] * sk_row_bcast<12>(nv_cur); pw[5] = p[5] * sk_row_bcast<13>(nv_cur);
        pw[6] = p[6] * sk_row_bcast<14>(nv_cur); pw[7] = p[7] * sk_row_bcast<15>(nv_cur);
      }
      if (dead != 0) {              // a row outside the context may hold anything as its norm
#pragma unroll
        for (int i = 0; i < 8; ++i)
          if (dead & (1u << i)) pw[i] = 0.f;
      }
      // weights as float16 hi + lo; columns [0,8) keep hi, columns [8,16) take the lo pair of the column
      // eight to their left
      union { sk_u32x4 u; uint32_t w[4]; } cv;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        auto h2 = __builtin_amdgcn_cvt_pkrtz(pw[2 * q], pw[2 * q + 1]);
        auto l2 = __builtin_amdgcn_cvt_pkrtz(pw[2 * q] - (float)h2[0], pw[2 * q + 1] - (float)h2[1]);
        union { decltype(h2) h; uint32_t u; } hb, lb;
        hb.h = h2;
        lb.h = l2;
        const uint32_t lo_left = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)lb.u, 0x118 /*row_shr:8*/, 0xf, 0xf, true);
        cv.w[q] = col < 8 ? hb.u : lo_left;
      }
      l_run = l_run * resc + psum;
      const float resc_left = sk_from_lo_cols(resc);
      const float resc_out = col < 8 ? resc : resc_left;
      const uint32_t par = F & 1u;
      *(sk_lds_u128*)(uintptr_t)(pb_addr + PB_PAR * par) = cv.u;
      *(sk_lds_u32*)(uintptr_t)(rs_addr + RS_PAR * par) = __float_as_uint(resc_out);
      sk_publish(cnt_written, F + 1u);
      if (last) {
        const float lsum = sk_rows_sum(l_run);
        if (col < gqa && g == 0) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (hs * gqa + col);
          a.part_ml[slot * 2] = m_run * 0.6931471805599453f;   // back to the natural-log domain
          a.part_ml[slot * 2 + 1] = lsum;
        }
        if (cw.valid) {
          s = cw.s; nchunks = cw.nchunks; nblk = cw.nblk; blk_lo = cw.blk_lo;
          walk_begin(cw);
          ctx = akv_seq_tokens(context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
          t_end = (int)min((int64_t)(blk_lo + nblk) * bs, ctx);
        }
        c = 0;
        m_run = -INFINITY;
        l_run = 0.f;
      } else {
        ++c;
      }
    }
  } else {
    // =========================== value wavefront ===========================
    // reader: lane (dword m = col, tokens 4 g + i): dword col of row (4 g + i, hs); token i lies i * 512 bytes on,
    // tile 1 another 8192
    const uint32_t vaddr = SK_VRING + (uint32_t)(4 * g) * 512u + (uint32_t)hs * 64u + (uint32_t)col * 4u;
    sk_float4 o[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (sk_float4){0.f, 0.f, 0.f, 0.f};

    // chunks 0..2 have landed (waited for before the table was written); copy chunk 0
    sk_publish(cnt_landed, 3u);
    sk_wait_progress(cnt_poll, lane < 8 ? 1u : 0u, status, limit);
    uint32_t v[8];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) v[4 * j + i] = *(sk_lds_cu32*)(uintptr_t)(vaddr + (uint32_t)j * SK_TILE + (uint32_t)i * 512u);
    sk_publish(cnt_copied, 1u);
    uint32_t r_slot = 1;

    for (uint32_t F = 0; F < N; ++F) {
      const bool last = c == nchunks - 1;
      const bool more = F + 1u < N;
      const uint32_t par = F & 1u;
      // ---- back stage, everything of chunk F that needs no weights: pairs of tokens (2p, 2p+1) of this lane's
      // eight -> bytes of (even | odd) coordinates, and all 32 lookups
      uint32_t xe[4], xo[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const uint32_t wa = v[2 * p], wb = v[2 * p + 1];
        xe[p] = (wa & 0xF0F0F0F0u) | ((wb >> 4) & 0x0F0F0F0Fu);
        xo[p] = ((wa << 4) & 0xF0F0F0F0u) | (wb & 0x0F0F0F0Fu);
      }
      uint32_t wv[8][4];    // M-tile n: byte n / 2 of the dword, even (xe) or odd (xo) coordinate
#pragma unroll
      for (int n = 0; n < 8; ++n)
#pragma unroll
        for (int p = 0; p < 4; ++p) wv[n][p] = sk_lut(lanebits, (n & 1) ? xo[p] : xe[p], SK_SEL(n >> 1));
      __builtin_amdgcn_sched_barrier(0);
      // ---- front stage.  Chunk F + 1 is complete in LDS, everybody has copied chunk F out of the slot that the
      // loads of chunk F + 3 are about to overwrite, and the score wavefront of this head has written the weights
      // of chunk F.
      sk_wait_progress(cnt_poll, lane < 8 ? (more ? F + 2u : 0u) : (lane < 16 ? F + 1u : (lane == 16 ? F + 1u : 0u)), status, limit);
      union { sk_half8 h; sk_u32x4 u; } cv;
      cv.u = *(sk_lds_u128*)(uintptr_t)(pb_addr + PB_PAR * par);
      const float resc = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(rs_addr + RS_PAR * par));
      if (more) {
        const uint32_t slot_off = r_slot * SK_SLOT;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) v[4 * j + i] = *(sk_lds_cu32*)(uintptr_t)(vaddr + slot_off + (uint32_t)j * SK_TILE + (uint32_t)i * 512u);
        r_slot = r_slot == 2 ? 0 : r_slot + 1;
        asm volatile("" ::: "memory");
        // queued behind the reads: executed once they have fetched their data; the score wavefront of the head
        // reads it as "the weights of chunk F are taken"
        sk_publish(cnt_copied, F + 2u);
      }
      __builtin_amdgcn_sched_barrier(0);
      issue();                        // chunk F + 3 into the slot of chunk F
      __builtin_amdgcn_sched_barrier(0);
      // this wavefront's loads of chunk F + 2 have landed (2 newer instructions: chunk F + 3)
      SK_WAIT_VM(2);
      sk_publish(cnt_landed, F + 3u);
      __builtin_amdgcn_sched_barrier(0);
      if (__builtin_amdgcn_ballot_w64(resc != 1.f) != 0) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[j][i] *= resc;
      }
#pragma unroll
      for (int n = 0; n < 8; ++n)
        o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sk_pack(wv[n][0], wv[n][1], wv[n][2], wv[n][3]), cv.h, o[n], 0, 0, 0);
      if (last) {
        // columns [0,8) + [8,16); lane (col < gqa, g) holds coordinates 32 g + 8 i + (M-tile j)
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[j][i] = (o[j][i] + sk_from_hi_cols(o[j][i])) * inv_alpha;
        if (col < gqa) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (hs * gqa + col);
          float* dst = a.part_acc + slot * 128 + 32 * g;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            *(float4*)(dst + 8 * i) = make_float4(o[0][i], o[1][i], o[2][i], o[3][i]);
            *(float4*)(dst + 8 * i + 4) = make_float4(o[4][i], o[5][i], o[6][i], o[7][i]);
          }
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (sk_float4){0.f, 0.f, 0.f, 0.f};
        if (cw.valid) {
          s = cw.s; nchunks = cw.nchunks; nblk = cw.nblk; blk_lo = cw.blk_lo;
          walk_begin(cw);
        }
        c = 0;
      } else {
        ++c;
      }
    }
  }
  SK_WAIT_VM(0);     // the loads issued past the end of the range land before the workgroup's LDS is released
}

__global__ __launch_bounds__(SK_THREADS) void akv_attn_stream_kernel(
    akv_attn_args a, akv_stream_extra x, const int32_t* __restrict__ prefix,
    const void* __restrict__ block_tables, const void* __restrict__ context_lens, const int32_t* __restrict__ wgdesc) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  if ((wave >> 3) == 0) sk_role_main<0>(a, x, prefix, block_tables, context_lens, wgdesc, wave & 7);
  else sk_role_main<1>(a, x, prefix, block_tables, context_lens, wgdesc, wave & 7);
}

// ----------------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------------
int akv_attn_spin_limit();      // akv_attn_mfma.hip

// Which matrix-core kernel serves the dense eight-head 4-bit layout: 0 = the one with register loads
// (akv_attn_mfma.hip), 1 = this one.  Sustained back-to-back calls run both at the same speed (84 us at the
// benchmark shape); in short bursts and single calls this one is 6-10 % slower, so it is not the default.
// AKV_ATTN_STREAM=1 in the environment or akv_debug_set_attn_stream(1) selects it.
static int g_stream_mode = -1;
static bool stream_enabled() {
  if (g_stream_mode < 0) {
    const char* e = getenv("AKV_ATTN_STREAM");
    g_stream_mode = (e && e[0] == '1') ? 1 : 0;
  }
  return g_stream_mode == 1;
}
extern "C" int akv_debug_set_attn_stream(int on) {
  g_stream_mode = on ? 1 : 0;
  return AKV_OK;
}

size_t akv_attn_stream_extra_bytes(int S) { return akv_align256((size_t)S * 8 * 8 * 64 * 16); }

// dense 4-bit cache of 8 kv heads: codes [blocks][bs][8][64], norms [blocks][bs][8], 16-byte aligned blocks
bool akv_attn_stream_applicable(const akv_attn_args& a, int d, int bits) {
  if (!stream_enabled()) return false;
  if (d != 128 || bits != 4 || (a.block_size != 16 && a.block_size != 32)) return false;
  if (a.KVH != 8 || a.QH % 8 != 0 || a.QH / 8 > 8) return false;
  if (a.num_blocks >= ((int64_t)1 << 31)) return false;
  const int64_t tile = (int64_t)a.block_size * 512;
  if (a.kps_head != 64 || a.kps_pos != 512 || a.kps_blk < tile || a.kps_blk >= ((int64_t)1 << 31) || (a.kps_blk & 15)) return false;
  if (a.vps_head != 64 || a.vps_pos != 512 || a.vps_blk < tile || a.vps_blk >= ((int64_t)1 << 31) || (a.vps_blk & 15)) return false;
  const int64_t ntile = (int64_t)a.block_size * 8;
  if (a.kns_head != 1 || a.kns_pos != 8 || a.kns_blk < ntile || a.kns_blk >= ((int64_t)1 << 31) || (a.kns_blk & 3)) return false;
  if (a.vns_head != 1 || a.vns_pos != 8 || a.vns_blk < ntile || a.vns_blk >= ((int64_t)1 << 31) || (a.vns_blk & 3)) return false;
  if ((((uintptr_t)a.kp | (uintptr_t)a.vp | (uintptr_t)a.kn | (uintptr_t)a.vn) & 15) != 0) return false;
  if (!a.kp || !a.vp || !a.kn || !a.vn || a.max_blocks_per_seq <= 0 || a.num_blocks <= 0) return false;   // block 0 must exist
  return true;
}

int akv_attn_stream_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* PiT,
                        const akv_attn_args& a, int bits, const akv_attn_ws& ws, void* extra_ws, int grid, hipStream_t stream) {
  akv_stream_extra x;
  x.lut = ws.lut;
  x.qop = (const uint4*)extra_ws;
  x.status = ws.status;
  x.spin_limit = akv_attn_spin_limit();
  const float qscale = a.scale * 1.4426950408889634f;   // scores come out in the log2 domain
  const int pgrid = a.S * a.KVH + 2;
#define SK_PRO(DT) akv_attn_stream_prologue_kernel<DT><<<pgrid, 256, 0, stream>>>(query, qs_seq, qs_head, PiT, a.centroids, a.S, a.QH, a.KVH, a.context_lens, a.cl_itype, a.block_size, a.max_blocks_per_seq, ws.prefix, (uint4*)x.qop, (uint32_t*)x.lut, ws.status, ws.wgdesc, grid, qscale, bits)
  if (q_dtype == AKV_F16) SK_PRO(AKV_F16); else if (q_dtype == AKV_BF16) SK_PRO(AKV_BF16); else SK_PRO(AKV_F32);
#undef SK_PRO
  AKV_LAUNCH_CHECK("akv_attn_stream_prologue_kernel");
  static bool configured = false;
  if (!configured) {
    AKV_HIP(hipFuncSetAttribute((const void*)akv_attn_stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS_BYTES));
    configured = true;
  }
  AKV_LAUNCH_TIMED(akv_attn_stream_kernel, grid, SK_THREADS, SK_LDS_BYTES, stream, a, x, ws.prefix, a.block_tables,
                   a.context_lens, ws.wgdesc);
  AKV_LAUNCH_CHECK("akv_attn_stream_kernel");
  return AKV_OK;
}
