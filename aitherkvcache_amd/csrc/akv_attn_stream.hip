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
// Chunks of 32 tokens (two tiles) flow through two rings of three slots (K and V).  A wavefront waits
// for its own loads of a chunk (s_waitcnt vmcnt with a count: every issue step emits the same number
// of vector-memory instructions, real or dummy, so the count is a constant), says so in an arrival
// counter, waits until all eight wavefronts of its role have said so, copies its head's rows into
// registers, says so in a done counter, and issues the loads of the chunk two ahead into the slot that
// all eight have finished reading.  Register layouts, the byte-pair lookup table (one table of
// fp16(alpha c) pairs serves K and V; 1 / alpha rides in the query operand and in the final scale),
// the softmax in the log2 domain and the weight hand-off are those of akv_attn_mfma.hip.
//
// LDS map (160 KB): [0, 64 KB) table region, entry e at e * 256: 32 copies of the fp16 pair in the
// first 128 bytes (a lookup is byte * 256 + (lane & 31) * 4, conflict-free), the second 128 bytes are
// "fragment e", used for the weight exchange (20 fragments per head), the norm tiles (one fragment per
// 4 tokens x 8 heads) and the counters; [64 KB, 112 KB) K ring; [112 KB, 160 KB) V ring.
// Inside a ring slot a tile keeps the cache's own order [token][head][64 bytes], except that the eight
// 16-byte pieces of every 128-byte line are stored at position (piece ^ (token & 7)): the loader lane
// that lands at position p fetches piece p ^ (token & 7) (its eight neighbours still cover the whole
// line), and the readers -- lane (token n, quarter g) of a score wavefront reading 16 bytes, lane
// (dword m, tokens 4g..4g+3) of a value wavefront reading dwords -- meet no bank conflicts.
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
#define SK_F_CNT 208                         // arriveK[8] | arriveV[8] | doneK[8] | doneV[8]
#define SK_F_FLAG 209                        // per head: ready, done (8 bytes)
#define SK_F_DUMP 210                        // target of the dummy loads
#define SK_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0f70 | (n))   // vmcnt(n), n < 16; other counters untouched
#define SK_W_VHI 512                         // words of the cached table block (as akv_attn_mfma.hip)
#define SK_W_TAG 768
#define SK_W_MARK 784
#define SK_W_ALPHA 785
#define SK_MARK 0x9100u                     // differs from the marker of akv_attn_mfma.hip, whose block holds more tables
#define SK_ALPHA_CANDIDATES 65536

struct akv_stream_extra {
  const uint32_t* lut;
  const uint4* qop;       // [S][8 heads][4 k-steps][64 lanes] half8
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
    uint4* __restrict__ qop, uint32_t* __restrict__ lut, uint32_t* __restrict__ status, float qscale, int bits) {
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
    // the words the other matrix-core kernel keeps in this block are rebuilt by it when it runs: drop its marker
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
  // operand of k-step st: lane (col, g), element e = coordinate 32 g + kcoord(st, e / 2, e % 2); columns
  // [0,8) hold the fp16 rounding of q', columns [8,16) the fp16 of the remainder
  {
    const int st = tid >> 6, lane = tid & 63;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int d = 32 * g + (bits == 4 ? mf_kcoord<4>(st, e >> 1, e & 1) : bits == 3 ? mf_kcoord<3>(st, e >> 1, e & 1) : mf_kcoord<2>(st, e >> 1, e & 1));
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
    qop[((size_t)(s * KVH + h) * 4 + st) * 64 + lane] = o;
  }
}

// ----------------------------------------------------------------------------------
// main kernel helpers
// ----------------------------------------------------------------------------------
#define SK_SEL(k) (0x0c020400u + ((uint32_t)(k) << 8))
// table lookup: address = byte k of `word` * 256 + lanebits, one byte permute
__device__ __forceinline__ uint32_t sk_lut(uint32_t lanebits, uint32_t word, uint32_t sel) {
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
__device__ __forceinline__ void sk_dma4(const void* src, uint32_t lds_dst) {
  __builtin_amdgcn_global_load_lds((sk_glb_ptr)src, (sk_lds_ptr)(uintptr_t)lds_dst, 4, 0, 0);
}

// Bounded waits on LDS counters.  LDS operations of a wavefront execute in order, so a counter written
// after data is seen after the data.  A wait that gives up marks the call (vector store); the reduce
// kernel then turns every output into NaN.
__device__ __forceinline__ void sk_give_up(uint32_t* status) {
  if ((threadIdx.x & 63) == 0) *(volatile uint32_t*)status = AKV_STATUS_HANDOFF_TIMEOUT;
}
__device__ __forceinline__ void sk_wait_ge(uint32_t addr, uint32_t need, uint32_t* status, int limit) {
  for (int spin = 0; spin < limit; ++spin) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    if ((int32_t)((uint32_t)__builtin_amdgcn_readfirstlane((int)v) - need) >= 0) return;
    __builtin_amdgcn_s_sleep(1);
  }
  sk_give_up(status);
}
// all eight counters at addr8 (lane & 7 -> counter) have reached `need`
__device__ __forceinline__ void sk_wait_all8(uint32_t addr8, uint32_t need, uint32_t* status, int limit) {
  for (int spin = 0; spin < limit; ++spin) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr8) : "memory");
    if (__builtin_amdgcn_ballot_w64((int32_t)(v - need) < 0) == 0) return;
    __builtin_amdgcn_s_sleep(1);
  }
  sk_give_up(status);
}
__device__ __forceinline__ void sk_publish(uint32_t addr, uint32_t value) {
  asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");
}
// the same after every LDS read issued so far has returned its data
__device__ __forceinline__ void sk_publish_after_reads(uint32_t addr, uint32_t value) {
  asm volatile("s_waitcnt lgkmcnt(0)\n\tds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");
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
                                             const void* __restrict__ context_lens, const int hs) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const uint32_t lanebits = (uint32_t)(lane & 31) * 4u;
  uint32_t* const status = x.status;
  const int limit = x.spin_limit;
  // exchange of head slot hs: weights (16 bytes per lane) in fragments 20 hs + 8 par + lane / 8, rescale factors
  // (4 bytes per lane) in fragments 20 hs + 16 + 2 par + lane / 32; parity 1 lies a constant further on
  const uint32_t pb_addr = SK_FRAG(20 * hs + (lane >> 3)) + (uint32_t)(lane & 7) * 16u;
  const uint32_t rs_addr = SK_FRAG(20 * hs + 16 + (lane >> 5)) + (uint32_t)(lane & 31) * 4u;
  constexpr uint32_t PB_PAR = 8u * 256u, RS_PAR = 2u * 256u;
  const uint32_t fl_addr = SK_FRAG(SK_F_FLAG) + 8u * (uint32_t)hs;     // ready at +0, done at +4
  const uint32_t arrive_mine = SK_FRAG(SK_F_CNT) + 32u * ROLE + 4u * (uint32_t)hs;
  const uint32_t arrive_all = SK_FRAG(SK_F_CNT) + 32u * ROLE + 4u * (uint32_t)(lane & 7);
  const uint32_t done_mine = SK_FRAG(SK_F_CNT) + 64u + 32u * ROLE + 4u * (uint32_t)hs;
  const uint32_t done_all = SK_FRAG(SK_F_CNT) + 64u + 32u * ROLE + 4u * (uint32_t)(lane & 7);

  const bool bs32 = a.block_size == 32;
  const int bs = bs32 ? 32 : 16;
  const int G = gridDim.x;
  const int total = prefix[a.S];
  const int per = (total + G - 1) / G;
  const int g0 = blockIdx.x * per;
  const int g1 = min(total, g0 + per);
  if (g0 >= g1) return;
  const int gqa = a.QH / a.KVH;

  // ---- walk: first segment by bisection, later ones are the next sequences that own blocks
  auto walk_begin = [&](sk_walk& w, bool first) {
    if (w.gcur >= g1) { w.valid = false; return; }
    if (first) {
      w.s = akv_find_seq(prefix, a.S, w.gcur);
    } else {
      int s = w.s + 1;
      while (prefix[s + 1] <= w.gcur) ++s;      // sequences without blocks; stops before a.S because gcur < total
      w.s = s;
    }
    const int sb0 = prefix[w.s], sb1 = prefix[w.s + 1];
    w.blk_lo = w.gcur - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    w.nblk = blk_hi - w.blk_lo;
    w.nchunks = bs32 ? w.nblk : (w.nblk + 1) >> 1;
    w.gcur = sb0 + blk_hi;
    w.valid = true;
  };

  // ---- the loading side: one issue step per chunk, in walk order, always the same number of
  // vector-memory instructions (score role 4, value role 2)
  sk_walk lw;
  lw.gcur = g0; lw.s = 0; lw.valid = false;
  walk_begin(lw, true);
  int lc = 0;                 // chunk of the loader's segment
  uint32_t l_slot = 0;        // ring slot of the next issue step
  const unsigned char* const codes = ROLE == 0 ? a.kp : a.vp;
  const uint32_t cps_blk = (uint32_t)(ROLE == 0 ? a.kps_blk : a.vps_blk);
  const uint32_t ring = ROLE == 0 ? SK_KRING : SK_VRING;
  // loader lane -> (token 2 hs + lane / 32, 128-byte line (lane / 8) % 4, position lane % 8 holding piece position ^ (token & 7))
  const uint32_t ld_tok = 2u * (uint32_t)hs + (uint32_t)(lane >> 5);
  const uint32_t ld_voff = ld_tok * 512u + (uint32_t)((lane >> 3) & 3) * 128u + (((uint32_t)lane & 7u) ^ (ld_tok & 7u)) * 16u;
  const uint32_t tile1_off = bs32 ? 16u * 512u : 0u;
  // norm tiles (score role): wavefront hs brings tokens 4 (hs % 4) .. + 3 of tile hs / 4, lanes 0..7
  const int nj = hs >> 2, nq = hs & 3;
  const uint32_t nrm_voff = (uint32_t)nq * 32u + (uint32_t)(lane & 7) * 4u;      // floats
  const uint32_t nrm_tile1 = bs32 ? 128u : 0u;
  auto issue = [&]() {
    if (lw.valid) {
      const int bi = lw.blk_lo + (bs32 ? lc : 2 * lc);
      const int64_t row = (int64_t)lw.s * a.bt_stride + bi;
      const uint32_t p0 = (uint32_t)akv_clamp_block(akv_load_index(block_tables, a.bt_itype, row), a.num_blocks);
      uint32_t p1 = p0;
      if (!bs32 && 2 * lc + 1 < lw.nblk)
        p1 = (uint32_t)akv_clamp_block(akv_load_index(block_tables, a.bt_itype, row + 1), a.num_blocks);
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
      if (++lc == lw.nchunks) { lc = 0; walk_begin(lw, false); }
    } else {
      // past the end of the range: the same number of instructions, four bytes each into a dump fragment
      if (lane == 0) {
        sk_dma4(codes, SK_FRAG(SK_F_DUMP));
        sk_dma4(codes, SK_FRAG(SK_F_DUMP));
        if constexpr (ROLE == 0) {
          sk_dma4(codes, SK_FRAG(SK_F_DUMP));
          sk_dma4(codes, SK_FRAG(SK_F_DUMP));
        }
      }
    }
    l_slot = l_slot == 2 ? 0 : l_slot + 1;
  };

  // ---- the consuming side
  sk_walk cw;
  cw.gcur = g0; cw.s = 0; cw.valid = false;
  walk_begin(cw, true);
  uint32_t F = 0;             // chunks consumed so far (flat over segments)
  uint32_t c_slot = 0;

  if constexpr (ROLE == 0) {
    // =========================== score wavefront ===========================
    // reader: lane (token col, quarter g) -> 16 bytes of row (col, hs)
    const uint32_t kaddr = SK_KRING + (uint32_t)col * 512u + (uint32_t)(hs >> 1) * 128u +
                           ((((uint32_t)(hs & 1) * 4u + (uint32_t)g) ^ ((uint32_t)col & 7u)) * 16u);
    // norms of tokens 4 g + i: fragment (slot, array, tile, g), float [i][head]
    const uint32_t naddr = SK_FRAG(SK_F_NORM + g) + (uint32_t)hs * 4u;
    sk_half8 qb[4], qn[4];
    auto load_q = [&](sk_half8 (&dst)[4], int s) {
      const uint4* qp = x.qop + ((size_t)(s * a.KVH + hs) * 4) * 64 + lane;
#pragma unroll
      for (int st = 0; st < 4; ++st) {
        const uint4 u = qp[st * 64];
        dst[st] = sk_pack(u.x, u.y, u.z, u.w);
      }
    };
    __builtin_amdgcn_sched_barrier(0);
    load_q(qn, cw.s);
    __builtin_amdgcn_sched_barrier(0);
    issue();
    __builtin_amdgcn_sched_barrier(0);
    issue();
    __builtin_amdgcn_sched_barrier(0);

    while (cw.valid) {
      const int s = cw.s;
      const int nchunks = cw.nchunks, nblk = cw.nblk, blk_lo = cw.blk_lo;
      const int64_t ctx = akv_seq_tokens(context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
      const int t_end = (int)min((int64_t)(blk_lo + nblk) * bs, ctx);
      walk_begin(cw, false);                    // cw now describes the NEXT segment
      float m_run = -INFINITY, l_run = 0.f;
      for (int c = 0; c < nchunks; ++c) {
        // ---- this wavefront's loads of chunk F have landed (4 newer instructions: the next chunk's)
        SK_WAIT_VM(4);
        if (c == 0) {
#pragma unroll
          for (int st = 0; st < 4; ++st) qb[st] = qn[st];
        }
        sk_publish(arrive_mine, F + 1u);
        sk_wait_all8(arrive_all, F + 1u, status, limit);
        const uint32_t slot_off = c_slot * SK_SLOT;
        const uint32_t nslot = c_slot * 16u * 256u;       // 16 norm fragments per slot
        sk_u32x4 kraw[2];
        kraw[0] = *(sk_lds_u128*)(uintptr_t)(kaddr + slot_off);
        kraw[1] = *(sk_lds_u128*)(uintptr_t)(kaddr + slot_off + SK_TILE);
        float kn[8], vn[8];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            kn[4 * j + i] = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(naddr + nslot + (uint32_t)(j * 4) * 256u + (uint32_t)i * 32u));
            vn[4 * j + i] = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(naddr + nslot + (uint32_t)(8 + j * 4) * 256u + (uint32_t)i * 32u));
          }
        sk_publish_after_reads(done_mine, F + 1u);
        c_slot = c_slot == 2 ? 0 : c_slot + 1;
        // ---- queries of the next segment, requested a chunk before they are needed
        __builtin_amdgcn_sched_barrier(0);
        if (c == nchunks - 1 && cw.valid) load_q(qn, cw.s);
        // ---- loads of chunk F + 2 into the slot of chunk F - 1, once all eight have read that one
        if (F >= 1u) sk_wait_all8(done_all, F, status, limit);
        __builtin_amdgcn_sched_barrier(0);
        issue();
        __builtin_amdgcn_sched_barrier(0);

        // ---- scores: 8 k-steps (tile j, dword st), four table reads feed one MFMA
        float sv[8];
        {
          const uint32_t kw[8] = {kraw[0].x, kraw[0].y, kraw[0].z, kraw[0].w, kraw[1].x, kraw[1].y, kraw[1].z, kraw[1].w};
          uint32_t w[3][4];
          sk_float4 acc[2];
          acc[0] = (sk_float4){0.f, 0.f, 0.f, 0.f};
          acc[1] = (sk_float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int b = 0; b < 4; ++b) w[n][b] = sk_lut(lanebits, kw[n], SK_SEL(b));
#pragma unroll
          for (int n = 0; n < 8; ++n) {
            if (n + 2 < 8) {
#pragma unroll
              for (int b = 0; b < 4; ++b) w[(n + 2) % 3][b] = sk_lut(lanebits, kw[n + 2], SK_SEL(b));
            }
            acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sk_pack(w[n % 3][0], w[n % 3][1], w[n % 3][2], w[n % 3][3]),
                                                                 qb[n & 3], acc[n >> 2], 0, 0, 0);
          }
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) sv[4 * j + i] = (acc[j][i] + sk_from_hi_cols(acc[j][i])) * kn[4 * j + i];
        }
        if (c == nchunks - 1) {     // only the last chunk of a segment can hold masked tokens
          const int tok0 = blk_lo * bs + 32 * c;
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int tok = tok0 + 16 * j + 4 * g + i;
              const bool ok = (tok < t_end) && (j == 0 || bs32 || 2 * c + 1 < nblk);
              if (!ok) { sv[4 * j + i] = -INFINITY; vn[4 * j + i] = 0.f; }
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
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __builtin_amdgcn_exp2f(sv[i] - m_new);    // 0 for masked tokens
          psum += p;
          pw[i] = p * vn[i];
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
        // the buffer of this parity was last read for chunk F - 2
        const uint32_t par = F & 1u;
        if (F >= 2u) sk_wait_ge(fl_addr + 4u, F - 1u, status, limit);
        *(sk_lds_u128*)(uintptr_t)(pb_addr + PB_PAR * par) = cv.u;
        *(sk_lds_u32*)(uintptr_t)(rs_addr + RS_PAR * par) = __float_as_uint(resc_out);
        sk_publish(fl_addr, F + 1u);
        ++F;
      }
      float lsum = sk_rows_sum(l_run);
      if (col < gqa && g == 0) {
        const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (hs * gqa + col);
        a.part_ml[slot * 2] = m_run * 0.6931471805599453f;   // back to the natural-log domain
        a.part_ml[slot * 2 + 1] = lsum;
      }
    }
  } else {
    // =========================== value wavefront ===========================
    // reader: lane (dword m = col, tokens 4 g + i): dword of row (4 g + i, hs)
    uint32_t vaddr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t tok = 4u * (uint32_t)g + (uint32_t)i;
      vaddr[i] = SK_VRING + tok * 512u + (uint32_t)(hs >> 1) * 128u +
                 ((((uint32_t)(hs & 1) * 4u + (uint32_t)(col >> 2)) ^ (tok & 7u)) * 16u) + (uint32_t)(col & 3) * 4u;
    }
    const float inv_alpha = 1.f / __uint_as_float(x.lut[SK_W_ALPHA]);
    __builtin_amdgcn_sched_barrier(0);
    issue();
    __builtin_amdgcn_sched_barrier(0);
    issue();
    __builtin_amdgcn_sched_barrier(0);

    while (cw.valid) {
      const int s = cw.s;
      const int nchunks = cw.nchunks;
      walk_begin(cw, false);
      sk_float4 o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (sk_float4){0.f, 0.f, 0.f, 0.f};
      for (int c = 0; c < nchunks; ++c) {
        SK_WAIT_VM(2);
        sk_publish(arrive_mine, F + 1u);
        sk_wait_all8(arrive_all, F + 1u, status, limit);
        const uint32_t slot_off = c_slot * SK_SLOT;
        uint32_t v[8];
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) v[4 * j + i] = *(sk_lds_cu32*)(uintptr_t)(vaddr[i] + slot_off + (uint32_t)j * SK_TILE);
        sk_publish_after_reads(done_mine, F + 1u);
        c_slot = c_slot == 2 ? 0 : c_slot + 1;
        if (F >= 1u) sk_wait_all8(done_all, F, status, limit);
        __builtin_amdgcn_sched_barrier(0);
        issue();
        __builtin_amdgcn_sched_barrier(0);
        // pairs of tokens (2p, 2p+1) of this lane's eight -> bytes of (even | odd) coordinates
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
        const uint32_t par = F & 1u;
        sk_wait_ge(fl_addr, F + 1u, status, limit);
        union { sk_half8 h; sk_u32x4 u; } cv;
        cv.u = *(sk_lds_u128*)(uintptr_t)(pb_addr + PB_PAR * par);
        const float resc = __uint_as_float(*(sk_lds_cu32*)(uintptr_t)(rs_addr + RS_PAR * par));
        sk_publish_after_reads(fl_addr + 4u, F + 1u);
        if (__builtin_amdgcn_ballot_w64(resc != 1.f) != 0) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[j][i] *= resc;
        }
#pragma unroll
        for (int n = 0; n < 8; ++n)
          o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(sk_pack(wv[n][0], wv[n][1], wv[n][2], wv[n][3]), cv.h, o[n], 0, 0, 0);
        ++F;
      }
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
    }
  }
  SK_WAIT_VM(0);     // the loads issued past the end of the range land before the workgroup's LDS is released
}

__global__ __launch_bounds__(SK_THREADS) void akv_attn_stream_kernel(
    akv_attn_args a, akv_stream_extra x, const int32_t* __restrict__ prefix,
    const void* __restrict__ block_tables, const void* __restrict__ context_lens) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // table: thread (entry e, quarter qt) writes 8 of the entry's 32 copies
  {
    const int e = threadIdx.x >> 2, qt = threadIdx.x & 3;
    const uint32_t vhi = x.lut[SK_W_VHI + e];
    uint4* va = (uint4*)(lds_raw + e * 256 + qt * 32);
    va[0] = make_uint4(vhi, vhi, vhi, vhi);
    va[1] = make_uint4(vhi, vhi, vhi, vhi);
  }
  if (threadIdx.x < 32) {
    *(uint32_t*)(lds_raw + SK_FRAG(SK_F_CNT) + 4 * threadIdx.x) = 0u;
    if (threadIdx.x < 16) *(uint32_t*)(lds_raw + SK_FRAG(SK_F_FLAG) + 4 * threadIdx.x) = 0u;
  }
  __syncthreads();
  if ((wave >> 3) == 0) sk_role_main<0>(a, x, prefix, block_tables, context_lens, wave & 7);
  else sk_role_main<1>(a, x, prefix, block_tables, context_lens, wave & 7);
}

// ----------------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------------
int akv_attn_spin_limit();      // akv_attn_mfma.hip

static bool stream_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("AKV_DISABLE_STREAM");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

size_t akv_attn_stream_extra_bytes(int S) { return akv_align256((size_t)S * 8 * 4 * 64 * 16); }

// dense 4-bit cache of 8 kv heads: codes [blocks][bs][8][64], norms [blocks][bs][8], 16-byte aligned blocks
bool akv_attn_stream_applicable(const akv_attn_args& a, int d, int bits) {
  if (stream_disabled()) return false;
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
#define SK_PRO(DT) akv_attn_stream_prologue_kernel<DT><<<pgrid, 256, 0, stream>>>(query, qs_seq, qs_head, PiT, a.centroids, a.S, a.QH, a.KVH, a.context_lens, a.cl_itype, a.block_size, a.max_blocks_per_seq, ws.prefix, (uint4*)x.qop, (uint32_t*)x.lut, x.status, qscale, bits)
  if (q_dtype == AKV_F16) SK_PRO(AKV_F16); else if (q_dtype == AKV_BF16) SK_PRO(AKV_BF16); else SK_PRO(AKV_F32);
#undef SK_PRO
  AKV_LAUNCH_CHECK("akv_attn_stream_prologue_kernel");
  static bool configured = false;
  if (!configured) {
    AKV_HIP(hipFuncSetAttribute((const void*)akv_attn_stream_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS_BYTES));
    configured = true;
  }
  akv_profile_mark_begin(stream);
  akv_attn_stream_kernel<<<grid, SK_THREADS, SK_LDS_BYTES, stream>>>(a, x, ws.prefix, a.block_tables, a.context_lens);
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("akv_attn_stream_kernel");
  return AKV_OK;
}
