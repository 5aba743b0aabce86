// MFMA paged decode attention for the 4-, 3- and 2-bit caches at head_dim 128, block_size 16 or 32.
//
// One workgroup = 16 wavefronts working on one range of (sequence, block) pairs for all kv
// heads: wavefronts 0-7 are SCORE wavefronts (one per kv head), 8-15 VALUE wavefronts (same
// heads).  Tokens are taken 32 at a time (two physical blocks).  Per chunk a score wavefront
// loads the K codes and both norms, forms the scores on the matrix cores, updates the running
// softmax and leaves the weights (fp16 operand form) plus the rescale factor in LDS; after one
// workgroup barrier the value wavefront of the same head multiplies them into the value codes
// it prefetched meanwhile.  The two kinds overlap (the score side works on chunk c+1 while the
// value side consumes chunk c) and, at under 128 registers each, four wavefronts share a SIMD.
//
// Register layouts are chosen so that nothing is ever transposed:
//
//   scores   S^T[token, col] = sum_d Khat[token, d] * Qop[d, col]       v_mfma_f32_16x16x32_f16
//            A = Khat: lane (n = l%16, g = l/16) owns bytes [16g, 16g+16) of token n's code row
//            (one 16-byte load).  The k-slice of one MFMA is two code bytes = four coordinates,
//            each as (hi pair, lo pair): elements [hi c0, hi c1, lo c0, lo c1, hi c2, hi c3, lo c2,
//            lo c3], exactly two 8-byte table entries side by side.
//            B = Qop: the rotated, pre-scaled queries of the kv head's query heads with every
//            coordinate pair repeated to face the hi and the lo half; columns [0,8) = fp16 rounding
//            of q', columns [8,16) = fp16 of the remainder (q' to ~22 bits at no extra MFMA).
//            Result: lane (col, g) holds tokens 4g..4g+3 of the tile for column col.
//   softmax  running max / sum per query head in the log2 domain, on a PACKED copy of the scores: of the
//            sixteen columns only gqa (roundings) + gqa (remainders) carry sums, so the lanes of a row
//            share the eight tokens of a head -- four lanes a head (a token pair each) with at most four
//            query heads, two lanes (a tile each) with five to eight -- and exponentials and float16
//            splits are issued a quarter / half as often.  The weights p * |v| go back, by row shifts, to
//            where they are exactly the k-slice of the B operand of the next product (tokens 4g..4g+3 of
//            both tiles), again split hi / lo over columns [0,8) / [8,16).
//   values   O^T[coord, col] += sum_token Vhat[token, coord] * P[token, col]
//            A = Vhat^T: lane (m, g) loads dword m (coordinates 8m..8m+7) of its 8 tokens and
//            builds, for each of the 8 coordinates, the 8-token k-slice; M-tile j row m is
//            coordinate 8m + j.
//
// Dequantisation goes through tables in LDS.  4-bit: indexed by a whole BYTE, entry (a<<4|b) is the fp16
// pair (c[a], c[b]).  For K a byte holds two neighbouring coordinates of one token -- already a
// k-pair; a K entry is 8 bytes, the hi pair and the lo pair (c = hi + lo to ~22 bits), fetched by
// ONE LDS read (the LDS issues about one wavefront read per three to five cycles whatever its
// width, so an 8-byte read costs little more than a 4-byte one).  For V the k axis is the token axis, so bytes
// are first re-formed from the same nibble position of two neighbouring tokens (two bit-field
// inserts per 8 codes); the V table holds fp16(alpha c) with alpha in [1,2) chosen so that the
// sixteen levels are almost exactly representable, and alpha is divided out at the end.  Every
// table entry is replicated 32 times (address = entry * 256 + (lane & 31) * entry size), so lookups
// never conflict on a bank.
//
// The 3-bit and 2-bit caches index tables of their own shape with the packed bits as they lie in memory (no
// spreading to nibbles; the tq35 kernel below, whose parts mix code widths, does spread):
//   3-bit  a group of eight codes is a big-endian 24-bit word (one byte permute); an index is a 6-bit FIELD of it.
//          K: field = two neighbouring codes of a token, 64 entries of 8 bytes.  V: the codes at odd and at even
//          positions of two neighbouring tokens are merged into two words of four fields (three operations
//          each), 64 entries of 4 bytes.  An address costs two operations (field extract, shift-or) instead of
//          one byte permute.
//   2-bit  an index is a code BYTE.  K: four neighbouring codes of a token = the whole 16-byte A operand of one
//          MFMA (hi pair, lo pair, hi pair, lo pair), 16 copies per entry (a 16-byte read is served 16 lanes at a
//          time).  V: the same coordinate of FOUR tokens (tokens 4g, 4g+1 of both tiles, or 4g+2, 4g+3), 8-byte
//          entries, 32 copies; the four halfwords of a tile are loaded two to a register and merged by bit-field
//          inserts (16 operations for all 16 lookups of a chunk).  The weights are written in the same token
//          order.  With 64 KB + 64 KB of tables the exchange buffers live in a third region (160 KB in all).
// The order in which the coordinates reach the value product differs per format; it is undone for free by the order
// in which the accumulators are written out (mf_vtile).  The query operand is in natural coordinate order for all.
#include "akv_attn_common.h"
#include "akv_nibble.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

#define MF_HEADS 8                  // kv heads per pass = score wavefronts = value wavefronts
#define MF_THREADS 1024
#define MF_WAIT_VM0 0x0f70          // s_waitcnt vmcnt(0), other counters untouched
#define MF_WIN 30                   // chunks served by one window of 64 block ids (even, <= 31)
#define MF_LDS_BYTES (128 * 1024)   // two tables of 256 entries x 256 bytes
// entry e of table A at e*256:          [(hi pair, lo pair) for K x 32 copies]
// entry e of table B at 65536 + e*256:  [fp16(alpha c) pairs for V x 32 copies][128 bytes of exchange buffer]
#define MF_TABB 65536u
#define MF_XBUF 4096u                // distance of the two exchange buffers of a head slot
// exchange units of the kernel for the uniform formats: stride and start (4- and 3-bit: the spare halves of table B
// entries; 2-bit: 128-byte units after the tables)
#define MF_XSTRIDE(bits) ((bits) == 2 ? 128u : 256u)
#define MF_XBASE(bits) ((bits) == 2 ? 131072u : MF_TABB + 128u)
#define MF_LDS_BYTES_2BIT (160 * 1024)
#define MF_ALPHA_CANDIDATES 65536
// words of the table block kept in the workspace
#define MF_W_KHI 0
#define MF_W_KLO 256
#define MF_W_VHI 512
#define MF_W_TAG 768                // 16 centroids the tables were built from
#define MF_W_MARK 784
#define MF_W_ALPHA 785
#define MF_W_WORDS 1024
#define MF_MARK 0x7452u
static_assert(MF_W_WORDS * 4 <= AKV_WS_LUT_BYTES, "table block must fit the workspace header");

struct akv_mfma_extra {
  const uint32_t* lut;   // table block, MF_W_* (workspace header)
  const uint4* qop;      // [S][KVH][8 k-steps][64 lanes] half8 as uint4 (workspace)
  const int32_t* wgdesc; // [G][AKV_WGREC] record of every workgroup (workspace)
  uint32_t* status;      // status words of the call (workspace header)
  int spin_limit;        // polls a hand-off wait makes before it gives up
};

// ----------------------------------------------------------------------------------
// prologue: q' = Pi q in MFMA operand layout, block prefix, byte-pair table
// ----------------------------------------------------------------------------------
template <int QDT>
__global__ __launch_bounds__(256) void akv_attn_mfma_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const uint4* __restrict__ bop,
    const float* __restrict__ centroids, int S, int QH, int KVH, const void* context_lens,
    int cl_itype, int block_size, int64_t max_blocks_per_seq, int32_t* prefix,
    uint4* __restrict__ qop, uint32_t* __restrict__ lut, uint32_t* __restrict__ status, float qscale, int bits, int nqb,
    int32_t* __restrict__ wgdesc, int32_t* __restrict__ seqw, int G) {
  __shared__ __align__(16) float q_lds[8][132];   // [query head of the group][input coordinate], zero-padded heads
  __shared__ float qr_lds[8][132];     // (rows 4 banks apart: the eight heads of a coordinate are read together)
  __shared__ int32_t scratch[257];
  __shared__ float best_err[256];
  __shared__ float best_alpha[256];
  const int tid = threadIdx.x;
  // block 0: block prefix; block 1: tables (first, so that they start at once and do not wait for a free slot
  // behind the rotation blocks); blocks [2, 2 + nqb): query rotation, (sequence, kv head) items blockIdx.x - 2,
  // + nqb, ...
  const int nq = S * KVH;
  if ((int)blockIdx.x == 0) {
    if (tid == 0) status[0] = 0u;
    akv_attn_partition(prefix, S, G, block_size == 32 ? 1 : 2, wgdesc, seqw, scratch, context_lens, cl_itype, block_size,
                       max_blocks_per_seq);
    return;
  }
  if ((int)blockIdx.x == 1) {
    // The tables depend on the codebook only.  They are kept in the workspace together with
    // the centroids they were built from and a marker; when those match, nothing is rebuilt.
    __shared__ int stale;
    const int levels = 1 << bits;
    if (tid == 0) stale = (lut[MF_W_MARK] != MF_MARK + (uint32_t)bits) ? 1 : 0;
    __syncthreads();
    if (tid < levels && __float_as_uint(centroids[tid]) != lut[MF_W_TAG + tid]) stale = 1;
    __syncthreads();
    if (!stale) return;
    // alpha search: minimise the largest relative fp16 rounding error of alpha * c over the levels
    float c[16];
    for (int v = 0; v < 16; ++v) c[v] = centroids[v & (levels - 1)];
    float berr = 1e30f, balpha = 1.f;
    for (int k = 0; k < MF_ALPHA_CANDIDATES / 256; ++k) {
      const float al = 1.f + (float)(tid * (MF_ALPHA_CANDIDATES / 256) + k) / (float)MF_ALPHA_CANDIDATES;
      float worst = 0.f;
      for (int v = 0; v < 16; ++v) {
        const float x = al * c[v];
        const float r = __half2float(__float2half_rn(x));
        const float e = x != 0.f ? fabsf(r - x) / fabsf(x) : 0.f;
        worst = fmaxf(worst, e);
      }
      if (worst < berr) { berr = worst; balpha = al; }
    }
    best_err[tid] = berr;
    best_alpha[tid] = balpha;
    __syncthreads();
    if (tid == 0) {
      for (int t = 1; t < 256; ++t)
        if (best_err[t] < best_err[0]) { best_err[0] = best_err[t]; best_alpha[0] = best_alpha[t]; }
      lut[MF_W_ALPHA] = __float_as_uint(best_alpha[0]);
    }
    __syncthreads();
    const float al = best_alpha[0];
    // pair (high nibble, low nibble); nibble values above the top level do not occur
    const float c0 = centroids[(tid >> 4) & (levels - 1)], c1 = centroids[tid & 15 & (levels - 1)];
    const __half k0 = __float2half_rn(c0), k1 = __float2half_rn(c1);
    lut[MF_W_KHI + tid] = (unsigned)__half_as_ushort(k0) | ((unsigned)__half_as_ushort(k1) << 16);
    const __half l0 = __float2half_rn(c0 - __half2float(k0)), l1 = __float2half_rn(c1 - __half2float(k1));
    lut[MF_W_KLO + tid] = (unsigned)__half_as_ushort(l0) | ((unsigned)__half_as_ushort(l1) << 16);
    const __half v0 = __float2half_rn(al * c0), v1 = __float2half_rn(al * c1);
    lut[MF_W_VHI + tid] = (unsigned)__half_as_ushort(v0) | ((unsigned)__half_as_ushort(v1) << 16);
    if (tid < levels) lut[MF_W_TAG + tid] = __float_as_uint(centroids[tid]);
    __threadfence();
    __syncthreads();
    if (tid == 0) lut[MF_W_MARK] = MF_MARK + (uint32_t)bits;
    return;
  }
  const int gqa = QH / KVH;
  // q' = Pi q on the matrix cores: A = the queries of the kv head (row r = query head r % 8), B = the float16
  // hi + lo operand of the encode kernel (lane (col, g): output coordinate 8 col + N-tile, input coordinates
  // 32 g + 8 ks + e).  Wavefront w owns N-tiles 2w and 2w + 1; their operand registers are requested first and
  // stay for all items of the block.  (On the vector unit, with the queries broadcast from LDS, this kernel took
  // 23 us for 256 sequences x 8 kv heads.)
  const int lane = tid & 63, wave = tid >> 6;
  akv_half8 bh[2][4], bl[2][4];
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int idx = ((2 * wave + t) * 4 + ks) * 64 + lane;
      bh[t][ks] = akv_as_half8(bop[idx]);
      bl[t][ks] = akv_as_half8(bop[2048 + idx]);
    }
  for (int item = (int)blockIdx.x - 2; item < nq; item += nqb) {
  const int s = item / KVH, h = item % KVH;
  for (int i = tid; i < 8 * 128; i += 256) {
    const int q = i >> 7, j = i & 127;
    q_lds[q][j] = q < gqa ? akv_elem<QDT>::load(query, s * qs_seq + (h * gqa + q) * qs_head + j) : 0.f;
  }
  __syncthreads();
  {
    const int r = lane & 15, kg = lane >> 4;
    float v[4][8];
    float m = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const float4 x0 = *(const float4*)&q_lds[r & 7][32 * kg + 8 * ks];
      const float4 x1 = *(const float4*)&q_lds[r & 7][32 * kg + 8 * ks + 4];
      v[ks][0] = x0.x; v[ks][1] = x0.y; v[ks][2] = x0.z; v[ks][3] = x0.w;
      v[ks][4] = x1.x; v[ks][5] = x1.y; v[ks][6] = x1.z; v[ks][7] = x1.w;
#pragma unroll
      for (int e = 0; e < 8; ++e) m = fmaxf(m, fabsf(v[ks][e]));
    }
    const uint32_t ex = akv_row_exponent(akv_rows_max(m));
    const float sc = akv_row_scale(ex);
    akv_float4v acc[2];
    acc[0] = (akv_float4v){0.f, 0.f, 0.f, 0.f};
    acc[1] = (akv_float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      akv_half8 hi, lo;
      akv_split8(v[ks], sc, hi, lo);
      acc[0] = akv_mfma3(hi, lo, bh[0][ks], bl[0][ks], acc[0]);
      acc[1] = akv_mfma3(hi, lo, bh[1][ks], bl[1][ks], acc[1]);
    }
    // lane (col, kg) holds query heads 4 kg + i (kg < 2) at output coordinates 8 col + 2 wave and + 1
    const float usc = akv_row_unscale(ex) * (qscale / 64.f);     // lane q < 8: the factor of query head q
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float u0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(usc), i));
      const float u1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(usc), 4 + i));
      if (kg < 2) {
        const float ui = kg == 0 ? u0 : u1;
        qr_lds[4 * kg + i][8 * r + 2 * wave] = acc[0][i] * ui;
        qr_lds[4 * kg + i][8 * r + 2 * wave + 1] = acc[1][i] * ui;
      }
    }
  }
  __syncthreads();
  // operand layout: [k-step n][lane (col, g)][e]: coordinate 32g + 4n + 2(e/4) + e%2 -- the four coordinates
  // of k-step n are the two code bytes (4-bit), the two 6-bit fields (3-bit) or the one code byte (2-bit) the
  // score wavefront looks up for that step; elements 2,3 and 6,7 repeat 0,1 and 4,5: they face the lo
  // halves of the K table entries
  for (int n = tid >> 6; n < 8; n += 4) {
    const int lane = tid & 63;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int dim = 32 * g + 4 * n + 2 * (e >> 2) + (e & 1);
      float v = 0.f;
      if (col < 8) {
        if (col < gqa) v = __half2float(__float2half_rn(qr_lds[col][dim]));
      } else if (col - 8 < gqa) {
        const float full = qr_lds[col - 8][dim];
        v = full - __half2float(__float2half_rn(full));
      }
      hbits[e] = __half_as_ushort(__float2half_rn(v));
    }
    uint4 o;
    o.x = hbits[0] | (hbits[1] << 16); o.y = hbits[2] | (hbits[3] << 16);
    o.z = hbits[4] | (hbits[5] << 16); o.w = hbits[6] | (hbits[7] << 16);
    qop[((size_t)(s * KVH + h) * 8 + n) * 64 + lane] = o;
  }
  __syncthreads();     // q_lds and qr_lds are rewritten by the next item
  }
}

// ----------------------------------------------------------------------------------
// main kernel
// ----------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) const uint32_t mf_lds_cu32;
typedef __attribute__((address_space(3))) uint32_t mf_lds_u32;
typedef uint32_t mf_u32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) mf_u32x4 mf_lds_u128;

// The tables are the kernel's only LDS object, so they start at LDS address 0 and a table offset
// is the LDS address itself (saves one add per lookup).
// address = byte k of `word` * 256 + lanebits, built by one byte permute: result byte 0 <- lanebits
// byte 0 (the copy: (lane & 31) * entry size), byte 1 <- word byte k (selector 4 + k), byte 2 <-
// lanebits byte 2 (1 for the V table, which lies 65536 bytes up).
#define MF_SEL(k) (0x0c020400u + ((uint32_t)(k) << 8))
typedef uint32_t mf_u32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const mf_u32x2 mf_lds_cu64;

__device__ __forceinline__ uint32_t mf_lut(uint32_t lanebits, uint32_t word, uint32_t sel) {
  const uint32_t addr = __builtin_amdgcn_perm(word, lanebits, sel);
  return *(mf_lds_cu32*)(uintptr_t)addr;
}
// K lookup: (hi pair, lo pair) of one code byte
__device__ __forceinline__ mf_u32x2 mf_lut2(uint32_t lanebits, uint32_t word, uint32_t sel) {
  const uint32_t addr = __builtin_amdgcn_perm(word, lanebits, sel);
  return *(mf_lds_cu64*)(uintptr_t)addr;
}

// 2-bit K lookup: the whole A operand of one MFMA (four coordinates of one code byte, hi and lo pairs)
typedef __attribute__((address_space(3))) const mf_u32x4 mf_lds_cu128;
__device__ __forceinline__ mf_u32x4 mf_lut4(uint32_t lanebits, uint32_t word, uint32_t sel) {
  const uint32_t addr = __builtin_amdgcn_perm(word, lanebits, sel);
  return *(mf_lds_cu128*)(uintptr_t)addr;
}
// 3-bit lookups: the table index is a 6-bit field (two codes) of a 24-bit word; address = field * 256 + lanebits
__device__ __forceinline__ uint32_t mf_addr6(uint32_t lanebits, uint32_t word, int shift) {
  return (__builtin_amdgcn_ubfe(word, (uint32_t)shift, 6u) << 8) | lanebits;
}
// K lookup number b (0..3) of a code word: 4-bit byte b, 3-bit field b from the top of the 24-bit word
template <int BITS>
__device__ __forceinline__ mf_u32x2 mf_klook(uint32_t lanebits, uint32_t word, int b) {
  if constexpr (BITS == 3) return *(mf_lds_cu64*)(uintptr_t)mf_addr6(lanebits, word, 18 - 6 * b);
  else return mf_lut2(lanebits, word, MF_SEL(b));
}
// V lookup number k (0..3) of a regrouped word: 4-bit byte k, 3-bit field k from the bottom
template <int BITS>
__device__ __forceinline__ uint32_t mf_vlook(uint32_t lanebits, uint32_t word, int k) {
  if constexpr (BITS == 3) return *(mf_lds_cu32*)(uintptr_t)mf_addr6(lanebits, word, 6 * k);
  else return mf_lut(lanebits, word, MF_SEL(k));
}
// M-tile of the value product that holds coordinate k of the lane's eight (the order in which the regrouping
// of the code words hands the coordinates to the lookups)
template <int BITS>
__host__ __device__ constexpr int mf_vtile(int k) {
  if (BITS == 4) return k;
  if (BITS == 3) return 7 - k;
  constexpr int t2[8] = {6, 2, 4, 0, 7, 3, 5, 1};
  return t2[k];
}

__device__ __forceinline__ half8 mf_pack(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  union { uint32_t u[4]; half8 h; } x;
  x.u[0] = a; x.u[1] = b; x.u[2] = c; x.u[3] = d;
  return x.h;
}

// lane c receives the value of lane c + 8 of its row of 16 (zero for c >= 8)
__device__ __forceinline__ float mf_from_hi_cols(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x108 /*row_shl:8*/, 0xf, 0xf, true));
}
// lane c receives the value of lane c - 8 of its row (zero for c < 8)
__device__ __forceinline__ float mf_from_lo_cols(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x118 /*row_shr:8*/, 0xf, 0xf, true));
}

// block id x block stride on the scalar unit (a 64-bit product of 64-bit operands would go through
// the vector unit and drag the whole address into vector registers); strides are below 2^31
__device__ __forceinline__ uint64_t mf_umul(uint32_t a, uint32_t b) { return (uint64_t)a * (uint64_t)b; }

// Identity the optimiser cannot look through: keeps the widening of a 32-bit lane offset next to
// the load that uses it, where it folds into the (scalar base + 32-bit lane offset) address form
// instead of becoming a loop-invariant 64-bit register pair and a 64-bit add per load.
__device__ __forceinline__ uint32_t mf_here(uint32_t v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Reductions over the four 16-lane rows of a wavefront (every lane gets the result for its column)
// by the row-swap instructions: v_permlane32_swap exchanges rows {2,3} of its first operand with
// rows {0,1} of the second, v_permlane16_swap rows {1,3} with rows {0,2}; fed the same value twice
// they leave (rows 0,1,0,1 | rows 2,3,2,3) and (rows 0,0,2,2 | rows 1,1,3,3).  Two vector
// instructions per step, no trip through the LDS crossbar.
__device__ __forceinline__ float mf_rows_max(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float mf_rows_sum(float v) {
  auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Row shifts that write ONE bank (four neighbouring lanes) of every row of sixteen; the other lanes keep `old`.
// mf_to_bank<K>: lane 4K + c of a row receives `src` of lane c.
template <int K>
__device__ __forceinline__ float mf_to_bank(float old, float src) {
  static_assert(K >= 1 && K <= 3, "bank 0 holds its own values");
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src), 0x110 + 4 * K /*row_shr:4K*/, 0xf, 1 << K, false));
}
// mf_dpp_bank<CTRL, K>: lanes of bank K receive `src` through the row operation CTRL, the others keep `old`;
// mf_dpp_banks<CTRL, MASK>: the same for a set of banks
template <int CTRL, int K>
__device__ __forceinline__ float mf_dpp_bank(float old, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src), CTRL, 0xf, 1 << K, false));
}
template <int CTRL, int MASK>
__device__ __forceinline__ float mf_dpp_banks(float old, float src) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(old), __float_as_int(src), CTRL, 0xf, MASK, false));
}
template <int CTRL, int MASK>
__device__ __forceinline__ uint32_t mf_dpp_banks_u(uint32_t old, uint32_t src) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)old, (int)src, CTRL, 0xf, MASK, false);
}
// mf_pair_from_bank<Q>: lanes 0..3 of a row receive `hi` of lanes 4Q + c, lanes 8..11 receive `lo` of lanes 4Q + c,
// every other lane zero (quad_perm 0,1,2,3 is the shift by nothing)
template <int Q>
__device__ __forceinline__ uint32_t mf_pair_from_bank(uint32_t hi, uint32_t lo) {
  constexpr int hi_ctrl = Q == 0 ? 0xE4 : 0x100 + 4 * Q;                                            // row_shl:4Q
  constexpr int lo_ctrl = Q == 2 ? 0xE4 : (Q < 2 ? 0x110 + (8 - 4 * Q) : 0x100 + (4 * Q - 8));      // row_shr:8-4Q / row_shl:4Q-8
  int w = __builtin_amdgcn_update_dpp(0, (int)hi, hi_ctrl, 0xf, 0x1, false);
  w = __builtin_amdgcn_update_dpp(w, (int)lo, lo_ctrl, 0xf, 0x4, false);
  return (uint32_t)w;
}
// sum / maximum over the four banks of a row (every lane gets the result of the lanes c, c + 4, c + 8, c + 12)
__device__ __forceinline__ float mf_banks_max(float v) {
  v = fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124 /*row_ror:4*/, 0xf, 0xf, false)));
  return fmaxf(v, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128 /*row_ror:8*/, 0xf, 0xf, false)));
}
__device__ __forceinline__ float mf_banks_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x124 /*row_ror:4*/, 0xf, 0xf, false));
  return v + __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x128 /*row_ror:8*/, 0xf, 0xf, false));
}

// Pairwise hand-off between the score and the value wavefront of a head slot (tq35 kernel; the kernel
// for the uniform formats orders its chunks with workgroup barriers instead): two counters in LDS,
// `ready` (chunks whose weights are written) and `done` (chunks whose weights have been read), both
// counted from the start of the kernel.  LDS operations of a wavefront are executed in order, so a
// counter written after the data is seen after the data.  Waiting polls the counter with a short
// sleep; the wait is bounded, so every wavefront finishes whatever happens.  A wait that gives up
// leaves a mark in the status word of the call (an ordinary vector store): the kernel goes on with
// whatever the buffer holds, the reduce kernel turns every output of the call into NaN, and the host
// can read the word back (akv_paged_attn_status).
#define MF_SPIN_LIMIT (1 << 16)
__device__ __forceinline__ void mf_wait_ge(uint32_t addr, uint32_t need, uint32_t* status, int limit) {
  for (int spin = 0; spin < limit; ++spin) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(addr) : "memory");
    if ((int32_t)((uint32_t)__builtin_amdgcn_readfirstlane((int)v) - need) >= 0) return;
    __builtin_amdgcn_s_sleep(2);
  }
  if ((threadIdx.x & 63) == 0) *(volatile uint32_t*)status = AKV_STATUS_HANDOFF_TIMEOUT;
}
__device__ __forceinline__ void mf_publish(uint32_t addr, uint32_t value) {
  asm volatile("ds_write_b32 %0, %1" : : "v"(addr), "v"(value) : "memory");
}

// workgroup barrier that orders LDS traffic only (outstanding global loads keep flying)
__device__ __forceinline__ void mf_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

struct mf_kraw {       // score wavefront, one 32-token chunk
  uint4 k[2];          // K code rows: tile j, token l%16, the lane's quarter of the row (16 / 12 / 8 bytes)
  float nrm;           // one of the chunk's norms (any head of the pass; see the score role)
};
typedef uint32_t mf_u32x3 __attribute__((ext_vector_type(3)));
typedef uint16_t mf_u16x2 __attribute__((ext_vector_type(2)));
struct mf_vraw {       // value wavefront
  uint32_t v[8];       // V codes: token tau(g,e), the eight codes 8(l%16) .. 8(l%16)+7 (4 / 3 bytes); 2-bit: v[2j + i],
                       // tokens 4g + i (low half) and 4g + i + 2 (high half) of tile j, two bytes each
};

// What a wavefront starts from: the workgroup's record and the first window of block ids of its first segment
// (lane i: block blk_lo + i of the segment, clamped to the segment's last), fetched at the kernel's entry
struct mf_start {
  int g0, g1;              // the workgroup's range of the global block axis
  int s, sb0, sb1, ctx;    // first segment: sequence (-1: search the prefix), its first and one-past-last global block, its tokens
  int pbwin;
  uint32_t lutw[6];        // the words of the workspace's table block this thread turns into table entries (mf_fill_tables)
};

// The byte-pair tables (layout at MF_LDS_BYTES): thread (entry e, quarter qt) holds the entry's words (requested at
// the kernel's entry, before anything else) and writes 8 of its 32 copies with 16-byte stores.  The words of the
// workspace block are pairs indexed by two nibbles (first code << 4 | second code).
template <int BITS>
__device__ __forceinline__ void mf_load_table_words(const uint32_t* __restrict__ lut, uint32_t (&w)[6]) {
  const int e = threadIdx.x >> 2;
  if constexpr (BITS == 2) {
    // entry = one code byte.  K: four coordinates (codes from the top bits down) as (hi pair, lo pair) twice.
    // V: the same coordinate of four tokens (codes from the bottom bits up).
    const int k01 = ((e >> 6) << 4) | ((e >> 4) & 3), k23 = (((e >> 2) & 3) << 4) | (e & 3);
    const int v01 = ((e & 3) << 4) | ((e >> 2) & 3), v23 = (((e >> 4) & 3) << 4) | (e >> 6);
    w[0] = lut[MF_W_KHI + k01]; w[1] = lut[MF_W_KLO + k01]; w[2] = lut[MF_W_KHI + k23]; w[3] = lut[MF_W_KLO + k23];
    w[4] = lut[MF_W_VHI + v01]; w[5] = lut[MF_W_VHI + v23];
  } else {
    // 4-bit: entry = one code byte (two codes).  3-bit: entry = a 6-bit field, K (first code << 3 | second
    // code) of one token, V (code of the odd token << 3 | code of the even token) of one coordinate; 64 entries.
    int ke = e, ve = e;
    if constexpr (BITS == 3) {
      ke = (((e >> 3) & 7) << 4) | (e & 7);
      ve = ((e & 7) << 4) | ((e >> 3) & 7);
    }
    w[0] = lut[MF_W_KHI + ke]; w[1] = lut[MF_W_KLO + ke]; w[2] = lut[MF_W_VHI + ve];
    w[3] = 0u; w[4] = 0u; w[5] = 0u;
  }
}
template <int BITS>
__device__ __forceinline__ void mf_fill_tables(const uint32_t (&w)[6]) {
  const int e = threadIdx.x >> 2, qt = threadIdx.x & 3;
  mf_lds_u128* ka = (mf_lds_u128*)(uintptr_t)(uint32_t)(e * 256 + qt * 64);
  mf_lds_u128* va = (mf_lds_u128*)(uintptr_t)(uint32_t)(MF_TABB + e * 256 + qt * (BITS == 2 ? 64 : 32));
  if constexpr (BITS == 2) {
    // K: 16 copies of 16 bytes (this thread: copies 4qt .. 4qt+3); V: 32 copies of 8 bytes (copies 8qt .. 8qt+7)
#pragma unroll
    for (int i = 0; i < 4; ++i) ka[i] = (mf_u32x4){w[0], w[1], w[2], w[3]};
#pragma unroll
    for (int i = 0; i < 4; ++i) va[i] = (mf_u32x4){w[4], w[5], w[4], w[5]};
  } else if (BITS == 4 || e < 64) {
#pragma unroll
    for (int i = 0; i < 4; ++i) ka[i] = (mf_u32x4){w[0], w[1], w[0], w[1]};    // K copies 8qt .. 8qt+7 (8 bytes each)
#pragma unroll
    for (int i = 0; i < 2; ++i) va[i] = (mf_u32x4){w[2], w[2], w[2], w[2]};    // V copies 8qt .. 8qt+7 (4 bytes each)
  }
}

// One role of the pipeline (ROLE 0 = score wavefront, 1 = value wavefront).  The two roles are
// separate instantiations entered through one uniform branch, so that neither keeps the other's
// loop-invariant registers alive.
template <int ROLE, int BITS, int PACK>
__device__ __forceinline__ void mf_role_main(const akv_attn_args& a, const akv_mfma_extra& x, const int hs, const mf_start& st) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  // One workgroup barrier per chunk orders everything: in interval k the score wavefronts produce the
  // weights of chunk k into exchange buffer k % 2 while the value wavefronts, one interval behind, consume
  // chunk k - 1 from the other buffer.  The barrier also keeps the wavefronts of the eight heads on the
  // same tokens: the code rows of neighbouring heads share 64-byte memory sectors when a row is narrower
  // than a sector (48 bytes at 3 bits), and heads left to drift a few chunks apart fetch 40 % of those
  // sectors from memory twice; in step the kernel fetches 4 % more than the algorithmic bytes.  (Per-head
  // flag hand-offs through LDS instead of the barrier, polled by the waiting side, were 5 % slower at
  // 4 bits: every poll is an LDS round trip on the critical path of its wavefront.)
  constexpr bool SYNC = true;
  // the copy of a table entry a lane reads (2-bit: 16 copies of 16-byte K entries and 32 of 8-byte V entries, else
  // 32 copies of 8 and 4 bytes)
  const uint32_t lane4v = MF_TABB + (uint32_t)(lane & 31) * (BITS == 2 ? 8u : 4u);   // 2-bit: whole entries of table B, else their first halves
  const uint32_t lane4k = BITS == 2 ? (uint32_t)(lane & 15) * 16u : (uint32_t)(lane & 31) * 8u;               // table A
  // exchange buffers of this head slot: buffer b -> unit q = hs*2 + b = 16 entries' spare halves of table B
  //   weights (16 B per lane): entry 16q + lane/8, offset 128 + (lane%8)*16
  //   rescale (4 B per lane):  entry 16q + 8 + lane/32, offset 128 + (lane%32)*4
  // (buffer 1 lies 16 entries after buffer 0; the parity of the chunk is a compile-time constant
  // at every use, so it folds into the offset field of the LDS instruction)
  // (2-bit: the V entries fill table B, the exchange units are 128-byte entries of a region of their own after it)
  constexpr uint32_t XS = MF_XSTRIDE(BITS), XB0 = MF_XBASE(BITS), XPAR = 16u * XS;
  const uint32_t pb_addr = XB0 + (32u * hs + (uint32_t)(lane >> 3)) * XS + (uint32_t)(lane & 7) * 16u;
  const uint32_t rs_addr = XB0 + (32u * hs + 8u + (uint32_t)(lane >> 5)) * XS + (uint32_t)(lane & 31) * 4u;


  // blocks of 16 tokens: a chunk (32 tokens, two 16-token tiles) is two blocks; blocks of 32: one
  // block, its second tile 16 positions further in.  bs32 is the same in every wavefront.
  const bool bs32 = a.block_size == 32;
  const int bs = bs32 ? 32 : 16;
  // (the block prefix of the batch in a register, one entry per lane: finding a segment's sequence and its
  // bounds costs no chain of dependent loads)
  const int held = akv_prefix_hold(a.prefix, a.S);
  // the workgroup's range of the global block axis, as the prologue cut it (whole workgroups per sequence
  // when the batch has few sequences, equal ranges otherwise)
  const int g0 = st.g0, g1 = st.g1;
  // the window of block ids: lane i of pbwin holds the physical id of block (2 * win_c0 + i) of the segment
  // (win_c0 + i for blocks of 32).  `fresh`: it holds window 0 of the first segment, from the kernel's entry.
  int pbwin = st.pbwin, win_c0 = 0;
  bool fresh = st.s >= 0;
  const int gqa = a.QH / a.KVH;
  // The tables are written by all wavefronts of the workgroup once, AFTER each has requested what its first chunks
  // need: the fill (LDS stores from registers and the barrier that publishes them) then runs beside those round
  // trips to memory instead of in front of them.
  bool filled = false;
  auto fill_once = [&]() {
    if (!filled) {
      mf_fill_tables<BITS>(st.lutw);
      mf_barrier();          // (orders LDS traffic only: the rows just requested keep flying)
      filled = true;
    }
  };

  int gcur = g0;
  while (gcur < g1) {
    // the first segment starts from the workgroup's record (scalar loads that the kernel's entry has already
    // brought in), later ones -- a range that crosses into the next sequence -- search the held prefix
    int s, sb0, sb1;
    int64_t ctx;
    if (gcur == g0 && st.s >= 0) {
      s = st.s;
      sb0 = st.sb0;
      sb1 = st.sb1;
      ctx = st.ctx;
    } else {
      s = akv_find_seq_held(a.prefix, a.S, held, gcur, sb0, sb1);
      ctx = akv_seq_tokens(a.context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
    }
    const int blk_lo = gcur - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    const int t_end = (int)min((int64_t)blk_hi * bs, ctx);
    gcur = sb0 + blk_hi;
    const int nblk = blk_hi - blk_lo;
    const int nchunks = bs32 ? nblk : (nblk + 1) >> 1;

    for (int hbase = 0; hbase < a.KVH; hbase += MF_HEADS) {
      const int h = hbase + hs;
      const bool active = h < a.KVH;
      // both wavefronts of an unused head slot skip the pass.  (A segment always has a chunk; saying so
      // here leaves ONE path into the chunk loops: were the first loads conditional, the compiler would
      // have to assume that the loads issued before them are the newest outstanding ones and would wait
      // for ALL loads, prefetches included, wherever the loop first touches their registers.)
      if (nchunks <= 0) continue;
      if (!active) {
        fill_once();
        if constexpr (SYNC)
          for (int i = 0; i <= nchunks; ++i) mf_barrier();     // the workgroup's barriers are counted by all
        continue;
      }
      const int hh = h;
      const int hd = a.hgroup > 1 ? h / a.hgroup : h;      // the head whose rows are read

      // physical block ids: lane i of pbwin holds the id of block (2 * win_c0 + i) of the segment
      // (win_c0 + i for blocks of 32).
      // A window of 64 ids serves MF_WIN chunks plus the two-chunk lookahead of the prefetch.  Its
      // reload drains every outstanding load (once per MF_WIN chunks); the chunk loop itself issues
      // the same loads on every path, so its waits stay counted waits for the chunk that is due.
      auto load_window = [&](int c0) {
        const int bi = min(blk_lo + (bs32 ? c0 : 2 * c0) + lane, blk_hi - 1);
        pbwin = (int)akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + bi), a.num_blocks);
        asm volatile("" : "+v"(pbwin));   // the window is complete here, not "maybe in flight" in the loop
        win_c0 = c0;
      };
      auto chunk_blocks = [&](int c_in, uint32_t& p0, uint32_t& p1) {
        const int c = min(c_in, nchunks - 1);      // lookahead past the end re-reads the last chunk
        const int w0 = bs32 ? c - win_c0 : 2 * (c - win_c0);
        const int w1 = (!bs32 && 2 * c + 1 < nblk) ? w0 + 1 : w0;
        p0 = (uint32_t)__builtin_amdgcn_readlane(pbwin, w0);
        p1 = (uint32_t)__builtin_amdgcn_readlane(pbwin, w1);
      };
      if (!fresh) load_window(0);
      fresh = false;

      if constexpr (ROLE == 0) {
        // =========================== score wavefront ===========================
        half8 qb[8];
        {
          const uint4* qp = x.qop + ((size_t)(s * a.KVH + hh) * 8) * 64 + lane;
#pragma unroll
          for (int st = 0; st < 8; ++st) {
            const uint4 u = qp[st * 64];
            qb[st] = mf_pack(u.x, u.y, u.z, u.w);
          }
        }
        float m_run = -INFINITY, l_run = 0.f;
        const uint32_t koff = (uint32_t)(hd * a.kps_head + col * a.kps_pos + (BITS == 4 ? 16 : BITS == 3 ? 12 : 8) * g);
        // Norms: the 32 K norms and 32 V norms a head needs per chunk lie 4 bytes apiece, one head stride apart.
        // Read per head they would be 64 addresses in sixteen or more 128-byte lines per load instruction; the
        // score wavefronts of the pass share the work instead: with n active head slots the 64 n norms of a
        // chunk are numbered [kind][token][head] and wavefront hs takes numbers 64 hs .. 64 hs + 63 (n = 8 and
        // dense norms: eight tokens x eight heads, two lines).  They are prefetched with the codes, written
        // into every head's exchange unit at the END of the step before the one that uses them (entries
        // 16q + 10 (K) and 16q + 11 (V) of the unit, 32 floats each) and read back after the barrier in the
        // accumulator layout.
        const int nact = min(MF_HEADS, a.KVH - hbase);
        const int nidx = 64 * hs + lane;
        const int nhead = nidx % nact, nrest = nidx / nact;
        const int ntok = nrest & 31;
        const bool nrm_is_v = nrest >= 32;
        const int nh = hbase + nhead;
        const int nhd = a.hgroup > 1 ? nh / a.hgroup : nh;
        const float* nrm_base = nrm_is_v ? a.vn : a.kn;
        const uint32_t nrm_blk = (uint32_t)(nrm_is_v ? a.vns_blk : a.kns_blk);
        const int npos = bs32 ? ntok : (ntok & 15);        // position of token ntok inside its block
        const uint32_t nrm_off = (uint32_t)(nrm_is_v ? nhd * a.vns_head + npos * a.vns_pos
                                                     : nhd * a.kns_head + npos * a.kns_pos);
        const uint32_t ktile1 = bs32 ? 16u * (uint32_t)a.kps_pos : 0u;   // second tile inside the same block
        const uint32_t nw_addr = XB0 + (32u * (uint32_t)nhead + 10u + (nrm_is_v ? 1u : 0u)) * XS + (uint32_t)ntok * 4u;
        const uint32_t nr_addr = XB0 + (32u * hs + 10u) * XS + (uint32_t)g * 16u;
        // (packed form, four lanes per head: the lane's bank kb = token pair, its two norms are eight of those sixteen
        // bytes; two lanes per head: kb = tile, all sixteen bytes of that tile)
        const int kb = PACK == 4 ? (lane >> 2) & 3 : (lane >> 3) & 1;
        const uint32_t nr2_addr = PACK == 4 ? nr_addr + 64u * (uint32_t)(kb >> 1) + 8u * (uint32_t)(kb & 1) : nr_addr + 64u * (uint32_t)kb;
        // what a lane hands over: a key norm as it is, a value norm as log2 |v| clamped below at -60 (a zero
        // vector then weighs 2^-60 of its codes: nothing at any output precision; NaN and negative norms,
        // which only rows outside a context can hold, come out as -60 as well)
        auto norm_out = [&](float n) { return nrm_is_v ? fmaxf(__builtin_amdgcn_logf(n), -60.f) : n; };
        auto load_chunk = [&](mf_kraw& r, int c) {
          uint32_t pb[2];
          chunk_blocks(c, pb[0], pb[1]);
          // the norm first: it is wanted one step before the rows, and loads complete in the order of issue
          r.nrm = nrm_base[mf_umul(ntok >= 16 ? pb[1] : pb[0], nrm_blk) + nrm_off];
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const unsigned char* kr = a.kp + mf_umul(pb[j], (uint32_t)a.kps_blk) + (j ? ktile1 : 0u) + mf_here(koff);
            if constexpr (BITS == 4) {
              r.k[j] = *(const uint4*)kr;
            } else if constexpr (BITS == 3) {
              const mf_u32x3 t = *(const mf_u32x3*)kr;
              r.k[j].x = t.x; r.k[j].y = t.y; r.k[j].z = t.z;
            } else {
              const uint2 t = *(const uint2*)kr;
              r.k[j].x = t.x; r.k[j].y = t.y;
            }
          }
        };
        // (`rn` holds the next chunk: its norms go out at the end of this step, behind the barrier that ends it)
        auto produce = [&](mf_kraw& r, const mf_kraw& rn, int c, const uint32_t par) {
          float sv[4];
          {
            // 8 steps of two MFMAs; the table reads of step n+2 are issued before the MFMAs of step n.
            //   4-bit: step = (tile j, dword st), 4 reads (one per code byte: hi and lo of two coordinates)
            //   3-bit: step = (tile j, group of 8 codes as a big-endian 24-bit word), 4 reads (one per 6-bit field)
            //   2-bit: step = (tile j, half of a dword), 2 reads (one per code byte: a whole MFMA operand)
            float4v acc[2];
            acc[0] = (float4v){0.f, 0.f, 0.f, 0.f};
            acc[1] = (float4v){0.f, 0.f, 0.f, 0.f};
            if constexpr (BITS == 2) {
              const uint32_t kw[4] = {r.k[0].x, r.k[0].y, r.k[1].x, r.k[1].y};
              mf_u32x4 w[3][2];
#pragma unroll
              for (int n = 0; n < 2; ++n)
#pragma unroll
                for (int b = 0; b < 2; ++b) w[n][b] = mf_lut4(lane4k, kw[n >> 1], MF_SEL(2 * (n & 1) + b));
#pragma unroll
              for (int n = 0; n < 8; ++n) {
                if (n + 2 < 8) {
#pragma unroll
                  for (int b = 0; b < 2; ++b) w[(n + 2) % 3][b] = mf_lut4(lane4k, kw[(n + 2) >> 1], MF_SEL(2 * (n & 1) + b));
                }
#pragma unroll
                for (int b = 0; b < 2; ++b)
                  acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                      mf_pack(w[n % 3][b].x, w[n % 3][b].y, w[n % 3][b].z, w[n % 3][b].w), qb[2 * (n & 3) + b], acc[n >> 2], 0, 0, 0);
              }
            } else {
              uint32_t kw[8];       // 4-bit: the code dwords; 3-bit: the 24-bit words
#pragma unroll
              for (int j = 0; j < 2; ++j) {
                if constexpr (BITS == 4) {
                  kw[4 * j + 0] = r.k[j].x; kw[4 * j + 1] = r.k[j].y; kw[4 * j + 2] = r.k[j].z; kw[4 * j + 3] = r.k[j].w;
                } else {
                  // group q = bytes 3q .. 3q+2 of the lane's twelve
                  kw[4 * j + 0] = __builtin_amdgcn_perm(r.k[j].x, r.k[j].x, 0x0c000102u);
                  kw[4 * j + 1] = __builtin_amdgcn_perm(r.k[j].y, r.k[j].x, 0x0c030405u);
                  kw[4 * j + 2] = __builtin_amdgcn_perm(r.k[j].z, r.k[j].y, 0x0c020304u);
                  kw[4 * j + 3] = __builtin_amdgcn_perm(r.k[j].z, r.k[j].z, 0x0c010203u);
                }
              }
              mf_u32x2 w[3][4];      // ring of three steps: two in flight behind the one multiplied
#pragma unroll
              for (int n = 0; n < 2; ++n)
#pragma unroll
                for (int b = 0; b < 4; ++b) w[n][b] = mf_klook<BITS>(lane4k, kw[n], b);
#pragma unroll
              for (int n = 0; n < 8; ++n) {
                if (n + 2 < 8) {
#pragma unroll
                  for (int b = 0; b < 4; ++b) w[(n + 2) % 3][b] = mf_klook<BITS>(lane4k, kw[n + 2], b);
                }
                acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    mf_pack(w[n % 3][0].x, w[n % 3][0].y, w[n % 3][1].x, w[n % 3][1].y), qb[2 * (n & 3)], acc[n >> 2], 0, 0, 0);
                acc[n >> 2] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                    mf_pack(w[n % 3][2].x, w[n % 3][2].y, w[n % 3][3].x, w[n % 3][3].y), qb[2 * (n & 3) + 1], acc[n >> 2], 0, 0, 0);
              }
            }
            __builtin_amdgcn_sched_barrier(0);   // not earlier: the loads reuse the registers just read
            load_chunk(r, c + 2);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (PACK == 2) {
              // Five to eight query heads per kv head: columns 0..7 carry the sums of the float16 roundings of the
              // queries, 8..15 those of their remainders.  The packed copy has two lanes per head: lane c keeps tile 0
              // (values 0..3), lane 8 + c takes tile 1 (values 4..7); each gets the other term of its tile from the
              // other lane by one row shift of eight that writes half of the row.
#pragma unroll
              for (int jj = 0; jj < 4; ++jj) {
                const float hi = mf_dpp_banks<0x118 /*row_shr:8*/, 0xc>(acc[0][jj], acc[1][jj]);
                const float lo = mf_dpp_banks<0x108 /*row_shl:8*/, 0x3>(acc[1][jj], acc[0][jj]);
                sv[jj] = hi + lo;
              }
            } else if constexpr (PACK == 4) {
              // At most four query heads per kv head: only columns 0..3 (the float16 roundings of the queries) and
              // 8..11 (their remainders) of a row of sixteen lanes carry sums, eight per lane.  Everything from
              // here to the weights runs on a PACKED copy instead: lane 4k + c of a row takes the token pair k
              // (values 2k, 2k + 1 of the eight) of head c -- the first term from lane c, the second from lane
              // 8 + c, by row shifts that write one bank of four lanes each.  Two sums, two norm products, four
              // exponentials (a quarter of the rate of ordinary vector instructions) and one float16 split per lane
              // and chunk in place of eight, eight, sixteen and four.
#pragma unroll
              for (int jj = 0; jj < 2; ++jj) {
                float hi = acc[0][jj];                                              // bank 0: its own values 0, 1
                hi = mf_dpp_bank<0x114 /*row_shr:4*/, 1>(hi, acc[0][2 + jj]);
                hi = mf_dpp_bank<0x118 /*row_shr:8*/, 2>(hi, acc[1][jj]);
                hi = mf_dpp_bank<0x11c /*row_shr:12*/, 3>(hi, acc[1][2 + jj]);
                float lo = acc[1][jj];                                              // bank 2: its own values 4, 5
                lo = mf_dpp_bank<0x108 /*row_shl:8*/, 0>(lo, acc[0][jj]);
                lo = mf_dpp_bank<0x104 /*row_shl:4*/, 1>(lo, acc[0][2 + jj]);
                lo = mf_dpp_bank<0x114 /*row_shr:4*/, 3>(lo, acc[1][2 + jj]);
                sv[jj] = hi + lo;
              }
            }
          }
          // The value norms arrive as log2 |v| (clamped below at -60, see the hand-over of the norms) and the
          // running maximum is kept over score + log2 |v|: the weight p |v| of a token is then exp2 of a
          // non-positive number, at most 1 whatever the size of the norms, and fits the float16 operand of the
          // value product with the same relative precision for tiny and for huge value vectors.  The
          // denominator sums the plain p = exp2(score - max) in the same frame (at most 2^60 each); the frame
          // cancels between numerator and denominator and travels as `m` of the partial result.
          float tv[4];
          if constexpr (PACK == 2) {
            // the lane's tile: four key norms and four log2 of value norms, sixteen bytes each
            union { mf_u32x4 u; float f[4]; } kn, vn;
            kn.u = *(mf_lds_u128*)(uintptr_t)(nr2_addr + XPAR * par);
            vn.u = *(mf_lds_u128*)(uintptr_t)(nr2_addr + XPAR * par + XS);
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              sv[jj] *= kn.f[jj];
              tv[jj] = sv[jj] + vn.f[jj];
            }
            if (c == nchunks - 1) {     // only the last chunk of a segment can hold masked tokens
              // (a row past the context may hold anything, NaN norms included: both sums are overwritten)
              const int tok0 = blk_lo * bs + 32 * c + 16 * kb + 4 * g;
              const bool tile_ok = kb == 0 || bs32 || 2 * c + 1 < nblk;
#pragma unroll
              for (int jj = 0; jj < 4; ++jj)
                if (!(tile_ok && tok0 + jj < t_end)) { sv[jj] = -INFINITY; tv[jj] = -INFINITY; }
            }
          } else {
            // the lane's token pair: key norms and log2 of the value norms, eight bytes each
            union { mf_u32x2 u; float f[2]; } kn, vn;
            kn.u = *(mf_lds_cu64*)(uintptr_t)(nr2_addr + XPAR * par);
            vn.u = *(mf_lds_cu64*)(uintptr_t)(nr2_addr + XPAR * par + XS);
#pragma unroll
            for (int jj = 0; jj < 2; ++jj) {
              sv[jj] *= kn.f[jj];
              tv[jj] = sv[jj] + vn.f[jj];
            }
            if (c == nchunks - 1) {     // only the last chunk of a segment can hold masked tokens
              // (a row past the context may hold anything, NaN norms included: both sums are overwritten)
              const int tok0 = blk_lo * bs + 32 * c + 16 * (kb >> 1) + 4 * g + 2 * (kb & 1);
              const bool tile_ok = (kb >> 1) == 0 || bs32 || 2 * c + 1 < nblk;
#pragma unroll
              for (int jj = 0; jj < 2; ++jj)
                if (!(tile_ok && tok0 + jj < t_end)) { sv[jj] = -INFINITY; tv[jj] = -INFINITY; }
            }
          }
          // running softmax in the log2 domain (scale * log2 e is folded into the query operand)
          union { mf_u32x4 u; uint32_t w[4]; } cv;
          float resc_out;
          if constexpr (PACK == 2) {
            // both lanes of a head agree on its running maximum; each keeps the sum of its own tile
            float mx = fmaxf(fmaxf(tv[0], tv[1]), fmaxf(tv[2], tv[3]));
            mx = fmaxf(mx, __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(mx), 0x128 /*row_ror:8*/, 0xf, 0xf, false)));
            mx = mf_rows_max(mx);
            const float m_new = fmaxf(m_run, mx);
            const float resc = __builtin_amdgcn_exp2f(m_run - m_new);   // 0 on the first chunk
            m_run = m_new;
            float psum = 0.f, pw[4];
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
              psum += __builtin_amdgcn_exp2f(sv[jj] - m_new);            // 0 for masked tokens
              pw[jj] = __builtin_amdgcn_exp2f(tv[jj] - m_new);           // p |v| <= 1; 0 for masked tokens
            }
            l_run = l_run * resc + psum;
            uint32_t hb[2], lb[2];      // the tile's two token pairs as float16 hi + lo
#pragma unroll
            for (int pp = 0; pp < 2; ++pp) {
              auto h2 = __builtin_amdgcn_cvt_pkrtz(pw[2 * pp], pw[2 * pp + 1]);
              auto l2 = __builtin_amdgcn_cvt_pkrtz(pw[2 * pp] - (float)h2[0], pw[2 * pp + 1] - (float)h2[1]);
              union { decltype(h2) h; uint32_t u; } hu, lu;
              hu.h = h2;
              lu.h = l2;
              hb[pp] = hu.u;
              lb[pp] = lu.u;
            }
            // operand dword qq = token pair q(qq) = pair q % 2 of tile q / 2: columns 0..7 take its hi form, columns
            // 8..15 its lo form, each from the lane of the pair's tile (its own, or the one eight lanes away)
            // (2-bit: the value side's operand takes the tokens as 4g, 4g+1 of both tiles, then 4g+2, 4g+3 of both)
            auto tile0 = [&](int pp) { return mf_dpp_banks_u<0x118 /*row_shr:8*/, 0xc>(hb[pp], lb[pp]); };
            auto tile1 = [&](int pp) { return mf_dpp_banks_u<0x108 /*row_shl:8*/, 0x3>(lb[pp], hb[pp]); };
            if constexpr (BITS == 2) {
              cv.w[0] = tile0(0); cv.w[1] = tile1(0); cv.w[2] = tile0(1); cv.w[3] = tile1(1);
            } else {
              cv.w[0] = tile0(0); cv.w[1] = tile0(1); cv.w[2] = tile1(0); cv.w[3] = tile1(1);
            }
            resc_out = resc;
          } else {
            // every lane of a row knows the running maximum of its head c; the sum is kept per lane (its own
            // pair's share) and added up over the banks when the segment ends
            float mx = fmaxf(tv[0], tv[1]);
            mx = mf_rows_max(mf_banks_max(mx));
            const float m_new = fmaxf(m_run, mx);
            const float resc = __builtin_amdgcn_exp2f(m_run - m_new);   // 0 on the first chunk
            m_run = m_new;
            const float psum = __builtin_amdgcn_exp2f(sv[0] - m_new) + __builtin_amdgcn_exp2f(sv[1] - m_new);   // 0 for masked tokens
            const float w0 = __builtin_amdgcn_exp2f(tv[0] - m_new), w1 = __builtin_amdgcn_exp2f(tv[1] - m_new);   // p |v| <= 1
            l_run = l_run * resc + psum;
            // the pair as float16 hi + lo (hi = truncated, lo = the exact float32 difference, truncated)
            auto h2 = __builtin_amdgcn_cvt_pkrtz(w0, w1);
            auto l2 = __builtin_amdgcn_cvt_pkrtz(w0 - (float)h2[0], w1 - (float)h2[1]);
            union { decltype(h2) h; uint32_t u; } hb, lb;
            hb.h = h2;
            lb.h = l2;
            // operand dword qq of a lane = token pair q(qq): columns 0..3 take the hi pair from bank q of their row,
            // columns 8..11 the lo pair; the other columns belong to no query head and hold zeros
            // (2-bit: the value side's operand takes the tokens as 4g, 4g+1 of both tiles, then 4g+2, 4g+3 of both)
            cv.w[0] = mf_pair_from_bank<0>(hb.u, lb.u);
            cv.w[1] = mf_pair_from_bank<BITS == 2 ? 2 : 1>(hb.u, lb.u);
            cv.w[2] = mf_pair_from_bank<BITS == 2 ? 1 : 2>(hb.u, lb.u);
            cv.w[3] = mf_pair_from_bank<3>(hb.u, lb.u);
            resc_out = resc;
          }
          // the buffer was last read for chunk c - 2, two barriers ago
          *(mf_lds_u128*)(uintptr_t)(pb_addr + XPAR * par) = cv.u;
          *(mf_lds_u32*)(uintptr_t)(rs_addr + XPAR * par) = __float_as_uint(resc_out);
          // the other parity's norm entries were last read in the step before this one
          *(mf_lds_u32*)(uintptr_t)(nw_addr + XPAR * (par ^ 1u)) = __float_as_uint(norm_out(rn.nrm));
        };

        mf_kraw ra, rb;
        __builtin_amdgcn_sched_barrier(0);     // the query operand is requested before the chunks
        load_chunk(ra, 0);
        __builtin_amdgcn_sched_barrier(0);     // queue order = chunk order, as in the loop
        load_chunk(rb, 1);
        __builtin_amdgcn_sched_barrier(0);
        fill_once();
        *(mf_lds_u32*)(uintptr_t)nw_addr = __float_as_uint(norm_out(ra.nrm));     // norms of chunk 0, ahead of the first barrier
        // pairs of chunks with the same loads on every path (an early exit from the middle of the
        // body would make the compiler wait for the newest prefetch at the top of every iteration)
        int c = 0;
        for (; c + 1 < nchunks; c += 2) {
          if (c - win_c0 >= MF_WIN) load_window(c);
          if constexpr (SYNC) mf_barrier();
          produce(ra, rb, c, 0);
          if constexpr (SYNC) mf_barrier();
          produce(rb, ra, c + 1, 1);
        }
        if (c < nchunks) {
          if constexpr (SYNC) mf_barrier();
          produce(ra, rb, c, 0);      // odd tail, already in ra
        }
        if constexpr (SYNC) mf_barrier();
        __builtin_amdgcn_s_waitcnt(MF_WAIT_VM0);   // the lookahead past the last chunk is never consumed
        float lsum = l_run;
        lsum = mf_rows_sum(lsum);
        // every lane of a row summed its own share
        if constexpr (PACK == 4) lsum = mf_banks_sum(lsum);
        else lsum += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(lsum), 0x128 /*row_ror:8*/, 0xf, 0xf, false));
        if (active && col < gqa && g == 0) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * gqa + col);
          a.part_ml[slot * 2] = m_run * 0.6931471805599453f;   // back to the natural-log domain
          a.part_ml[slot * 2 + 1] = lsum;
        }
      } else {
        // =========================== value wavefront ===========================
        float4v o[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (float4v){0.f, 0.f, 0.f, 0.f};
        // token 4g of a tile; the eight codes of coordinates 8 col .. 8 col + 7: one dword, three bytes
        // (taken from the aligned dword holding the first of them and, where they run over, from the
        // neighbour lane's dword), or one halfword
        const uint32_t voff = (uint32_t)(hd * a.vps_head + 4 * g * a.vps_pos + (BITS == 4 ? 4 * col : BITS == 3 ? ((3 * col) & ~3) : 2 * col));
        const uint32_t vtile1 = bs32 ? 16u * (uint32_t)a.vps_pos : 0u;     // second tile inside the same block
        const uint32_t o3 = (uint32_t)(3 * col) & 3u;
        const uint32_t sel3 = 0x0c000000u | (o3 << 16) | ((o3 + 1u) << 8) | (o3 + 2u);   // big-endian 24-bit word
        auto load_chunk = [&](mf_vraw& r, int c) {
          uint32_t pb[2];
          chunk_blocks(c, pb[0], pb[1]);
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const unsigned char* vb = a.vp + mf_umul(pb[j], (uint32_t)a.vps_blk) + (j ? vtile1 : 0u);
            if constexpr (BITS == 2) {
#pragma unroll
              for (int i = 0; i < 2; ++i) {
                union { mf_u16x2 h; uint32_t u; } t;
                t.h.x = *(const uint16_t*)(vb + (uint32_t)(i * (int)a.vps_pos) + mf_here(voff));
                t.h.y = *(const uint16_t*)(vb + (uint32_t)((i + 2) * (int)a.vps_pos) + mf_here(voff));
                r.v[2 * j + i] = t.u;
              }
            } else {
#pragma unroll
              for (int i = 0; i < 4; ++i) {    // the token step rides in the uniform base
                const unsigned char* vr = vb + (uint32_t)(i * (int)a.vps_pos) + mf_here(voff);
                r.v[4 * j + i] = *(const uint32_t*)vr;
              }
            }
          }
        };
        // Everything that does not need the weights happens BEFORE the barrier, while the score side
        // is still working: pairs of tokens (2p, 2p+1) of this lane's eight -> bytes of (even | odd)
        // coordinates, the raw registers take the chunk after next (see the score side), and all 32
        // table lookups of the chunk are issued.  After the barrier only the weights are read and
        // the eight MFMAs run back to back.
        // 4-bit and 3-bit: step n -> lookup n/2 of the regrouped word, even (xe) or odd (xo) position; M-tile n;
        // four lookups (pairs of tokens) make an operand.  2-bit: a lookup is one coordinate of FOUR tokens, two
        // make an operand; word n/2 of xe, bytes n%2 (tokens 4g, 4g+1 of both tiles) and n%2 + 2 (4g+2, 4g+3).
        uint32_t wv[4][4];
        uint32_t xe[4], xo[4];
        auto vlook = [&](uint32_t (&dst)[4], int n) {
          if constexpr (BITS == 2) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
              const mf_u32x2 t = mf_lut2(lane4v, xe[n >> 1], MF_SEL((n & 1) + 2 * p));
              dst[2 * p] = t.x;
              dst[2 * p + 1] = t.y;
            }
          } else {
#pragma unroll
            for (int p = 0; p < 4; ++p) dst[p] = mf_vlook<BITS>(lane4v, (n & 1) ? xo[p] : xe[p], n >> 1);
          }
        };
        auto regroup = [&](mf_vraw& r, int c) {
          if constexpr (BITS == 2) {
            // halves (a | c << 16) and (b | d << 16) of each tile: e = nibbles (a, b) of the codes at bit
            // positions 0 mod 4, o = those at 2 mod 4; then the nibbles of the two tiles side by side
            const uint32_t e0 = (r.v[0] & 0x33333333u) | ((r.v[1] << 2) & 0xccccccccu);
            const uint32_t o0 = ((r.v[0] >> 2) & 0x33333333u) | (r.v[1] & 0xccccccccu);
            const uint32_t e1 = (r.v[2] & 0x33333333u) | ((r.v[3] << 2) & 0xccccccccu);
            const uint32_t o1 = ((r.v[2] >> 2) & 0x33333333u) | (r.v[3] & 0xccccccccu);
            xe[0] = (e0 & 0x0f0f0f0fu) | ((e1 << 4) & 0xf0f0f0f0u);      // codes 3 and 7 of the lane's eight
            xe[1] = ((e0 >> 4) & 0x0f0f0f0fu) | (e1 & 0xf0f0f0f0u);      // codes 1 and 5
            xe[2] = (o0 & 0x0f0f0f0fu) | ((o1 << 4) & 0xf0f0f0f0u);      // codes 2 and 6
            xe[3] = ((o0 >> 4) & 0x0f0f0f0fu) | (o1 & 0xf0f0f0f0u);      // codes 0 and 4
          } else {
#pragma unroll
            for (int p = 0; p < 4; ++p) {
              uint32_t wa = r.v[2 * p], wb = r.v[2 * p + 1];
              if constexpr (BITS == 3) {
                // the lane's three bytes as a big-endian 24-bit word (code 0 in bits 23:21), then the codes at
                // odd positions (bits 0 mod 6) and at even positions (bits 3 mod 6) of the two tokens side by side
                const uint32_t na = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)wa, 0x101 /*row_shl:1*/, 0xf, 0xf, true);
                const uint32_t nb = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)wb, 0x101 /*row_shl:1*/, 0xf, 0xf, true);
                wa = __builtin_amdgcn_perm(na, wa, sel3);
                wb = __builtin_amdgcn_perm(nb, wb, sel3);
                xe[p] = (wa & 0x001c71c7u) | ((wb << 3) & 0x00e38e38u);
                xo[p] = ((wa >> 3) & 0x001c71c7u) | (wb & 0x00e38e38u);
              } else {
                xe[p] = (wa & 0xF0F0F0F0u) | ((wb >> 4) & 0x0F0F0F0Fu);
                xo[p] = ((wa << 4) & 0xF0F0F0F0u) | (wb & 0x0F0F0F0Fu);
              }
            }
          }
          __builtin_amdgcn_sched_barrier(0);   // not earlier: the loads reuse the registers just read
          load_chunk(r, c + 1);                // a whole chunk period ahead of its use
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int n = 0; n < 4; ++n) vlook(wv[n], n);
        };
        auto consume = [&](int c, const uint32_t par) {
          // second half of the lookups: in flight while the weights arrive and the first four MFMAs run
          uint32_t wl[4][4];
#pragma unroll
          for (int n = 4; n < 8; ++n) vlook(wl[n - 4], n);
          union { half8 h; mf_u32x4 u; } cv;
          cv.u = *(mf_lds_u128*)(uintptr_t)(pb_addr + XPAR * par);
          const float resc = __uint_as_float(*(mf_lds_cu32*)(uintptr_t)(rs_addr + XPAR * par));
          if (__builtin_amdgcn_ballot_w64(resc != 1.f) != 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
              for (int i = 0; i < 4; ++i) o[j][i] *= resc;
          }
#pragma unroll
          for (int n = 0; n < 4; ++n)
            o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(wv[n][0], wv[n][1], wv[n][2], wv[n][3]), cv.h, o[n], 0, 0, 0);
#pragma unroll
          for (int n = 4; n < 8; ++n)
            o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(wl[n - 4][0], wl[n - 4][1], wl[n - 4][2], wl[n - 4][3]), cv.h, o[n], 0, 0, 0);
        };

        auto step = [&](mf_vraw& r, int c, const uint32_t par) {
          regroup(r, c);
          consume(c, par);
        };
        mf_vraw ra;
        load_chunk(ra, 0);
        fill_once();
        if constexpr (SYNC) mf_barrier();
        for (int c = 0; c < nchunks; ++c) {
          if (c - win_c0 >= MF_WIN) load_window(c);
          if constexpr (SYNC) mf_barrier();
          step(ra, c, (uint32_t)(c & 1));
        }
        __builtin_amdgcn_s_waitcnt(MF_WAIT_VM0);
        // columns [0,8) + [8,16); lane (col < gqa, g) holds coordinates 32g + 8i + (coordinate of M-tile j)
        const float inv_alpha = 1.f / __uint_as_float(x.lut[MF_W_ALPHA]);
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) o[j][i] = (o[j][i] + mf_from_hi_cols(o[j][i])) * inv_alpha;
        if (active && col < gqa) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * gqa + col);
          float* dst = a.part_acc + slot * 128 + 32 * g;
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            *(float4*)(dst + 8 * i) = make_float4(o[mf_vtile<BITS>(0)][i], o[mf_vtile<BITS>(1)][i],
                                                  o[mf_vtile<BITS>(2)][i], o[mf_vtile<BITS>(3)][i]);
            *(float4*)(dst + 8 * i + 4) = make_float4(o[mf_vtile<BITS>(4)][i], o[mf_vtile<BITS>(5)][i],
                                                      o[mf_vtile<BITS>(6)][i], o[mf_vtile<BITS>(7)][i]);
          }
        }
      }
    }
  }
}

template <int BITS, int PACK>
__global__ __launch_bounds__(MF_THREADS) void akv_attn_mfma_kernel(akv_attn_args a, akv_mfma_extra x) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wavefront-uniform on purpose
  // ---- the workgroup's record (scalar loads) and, from it, the first window of 64 block ids of its first
  // segment: both requested here, ahead of the table fill, so that the two dependent trips to memory that every
  // wavefront would otherwise start with after the fill run beside it
  mf_start st;
  mf_load_table_words<BITS>(x.lut, st.lutw);      // (first: these loads depend on nothing)
  {
    const int32_t* rec = x.wgdesc + (size_t)blockIdx.x * AKV_WGREC;
    st.g0 = rec[AKV_WGREC_G0];
    st.g1 = rec[AKV_WGREC_G1];
    st.s = rec[AKV_WGREC_SEQ];
    st.sb0 = rec[AKV_WGREC_SB0];
    st.sb1 = rec[AKV_WGREC_SB1];
    st.ctx = rec[AKV_WGREC_CTX];
    st.pbwin = 0;
    if (st.g0 < st.g1 && st.s >= 0) {
      const int blk_lo = st.g0 - st.sb0, blk_hi = min(st.g1, st.sb1) - st.sb0;
      const int bi = min(blk_lo + (int)(threadIdx.x & 63), blk_hi - 1);
      st.pbwin = (int)akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, st.s * a.bt_stride + bi), a.num_blocks);
    }
  }
  if ((wave >> 3) == 0) mf_role_main<0, BITS, PACK>(a, x, wave & 7, st);
  else mf_role_main<1, BITS, PACK>(a, x, wave & 7, st);
}

// ----------------------------------------------------------------------------------
// host side
// ----------------------------------------------------------------------------------
static bool mfma_disabled() {
  static int v = -1;
  if (v < 0) {
    const char* e = getenv("AKV_DISABLE_MFMA");
    v = (e && e[0] == '1') ? 1 : 0;
  }
  return v == 1;
}

// extra workspace the MFMA path needs beyond akv_attn_ws (appended after it)
size_t akv_attn_mfma_extra_bytes(int S, int KVH) {
  return akv_align256((size_t)S * KVH * 8 * 64 * 16);
}

// polls a hand-off wait makes before it gives up (akv_debug_set_handoff_spin_limit)
static int g_spin_limit = MF_SPIN_LIMIT;
int akv_attn_spin_limit() { return g_spin_limit; }
extern "C" int akv_debug_set_handoff_spin_limit(int polls) {
  g_spin_limit = polls < 0 ? MF_SPIN_LIMIT : polls;
  return AKV_OK;
}

// query heads per kv head -> number of groups of at most eight the kv head is presented as (0: none fits)
static int akv_attn_mfma_head_groups(int gqa) {
  for (int hg = (gqa + 7) / 8; hg <= gqa && hg <= 8; ++hg)
    if (gqa % hg == 0) return hg;
  return 0;
}

bool akv_attn_mfma_applicable(const akv_attn_args& a, int d, int bits) {
  if (mfma_disabled()) return false;
  if (d != 128 || bits < 2 || bits > 4 || (a.block_size != 16 && a.block_size != 32)) return false;
  if (akv_attn_mfma_head_groups(a.QH / a.KVH) == 0) return false;
  if (a.num_blocks >= ((int64_t)1 << 31)) return false;                       // block ids travel as 32-bit lanes
  // K rows are read 16 / 12 / 8 bytes per lane, V rows by dword / dword / halfword.  Multi-dword
  // loads need dword alignment only, so the serving layout (rows of packed + 4 bytes: pitch 68 / 52 /
  // 36) qualifies as well as dense rows.
  const uintptr_t kalign = 3, valign = bits == 2 ? 1 : 3;
  if ((((uintptr_t)a.kp | (uintptr_t)a.kps_blk | (uintptr_t)a.kps_pos | (uintptr_t)a.kps_head) & kalign) != 0) return false;
  if ((((uintptr_t)a.vp | (uintptr_t)a.vps_blk | (uintptr_t)a.vps_pos | (uintptr_t)a.vps_head) & valign) != 0) return false;
  const int64_t strides[12] = {a.kps_blk, a.kps_pos, a.kps_head, a.kns_blk, a.kns_pos, a.kns_head,
                               a.vps_blk, a.vps_pos, a.vps_head, a.vns_blk, a.vns_pos, a.vns_head};
  for (int i = 0; i < 12; ++i)
    if (strides[i] < 0 || strides[i] >= ((int64_t)1 << 27)) return false;   // 32-bit in-block offsets
  // the largest in-block offset a lane forms (head, then position of the second tile, then the row) fits 32 bits
  const int64_t kmax = (int64_t)a.KVH * a.kps_head + 32 * a.kps_pos + 64, vmax = (int64_t)a.KVH * a.vps_head + 32 * a.vps_pos + 64;
  const int64_t nmax = (int64_t)a.KVH * (a.kns_head > a.vns_head ? a.kns_head : a.vns_head) + 32 * (a.kns_pos > a.vns_pos ? a.kns_pos : a.vns_pos);
  if (kmax >= ((int64_t)1 << 32) || vmax >= ((int64_t)1 << 32) || nmax >= ((int64_t)1 << 32)) return false;
  return true;
}

int akv_attn_mfma_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* PiT,
                      const akv_attn_args& a_in, int bits, const akv_attn_ws& ws, void* extra_ws, int grid, hipStream_t stream) {
  akv_attn_args a = a_in;
  a.hgroup = akv_attn_mfma_head_groups(a.QH / a.KVH);
  a.KVH *= a.hgroup;                        // from here on: groups of at most eight query heads
  int32_t* prefix = ws.prefix;
  akv_mfma_extra x;
  x.lut = ws.lut;
  x.qop = (const uint4*)extra_ws;
  x.wgdesc = ws.wgdesc;
  x.status = ws.status;
  x.spin_limit = g_spin_limit;
  const float qscale = a.scale * 1.4426950408889634f;   // scores come out in the log2 domain
  // rotation blocks: one per (sequence, kv head) up to six per CU (what its registers admit at once), then they loop
  const int cus = akv_cached_cu_count();
  const int nqb = a.S * a.KVH < 6 * (cus > 0 ? cus : 256) ? a.S * a.KVH : 6 * (cus > 0 ? cus : 256);
  const int pgrid = nqb + 2;
  const uint4* bop = (const uint4*)(PiT + 128 * 128);    // the encode kernel's operand follows Pi and PiT in the prepared buffer
#define MF_PRO(DT) akv_attn_mfma_prologue_kernel<DT><<<pgrid, 256, 0, stream>>>(query, qs_seq, qs_head, bop, a.centroids, a.S, a.QH, a.KVH, a.context_lens, a.cl_itype, a.block_size, a.max_blocks_per_seq, prefix, (uint4*)x.qop, (uint32_t*)x.lut, x.status, qscale, bits, nqb, ws.wgdesc, ws.seqw, grid)
  if (q_dtype == AKV_F16) MF_PRO(AKV_F16); else if (q_dtype == AKV_BF16) MF_PRO(AKV_BF16); else MF_PRO(AKV_F32);
#undef MF_PRO
  AKV_LAUNCH_CHECK("akv_attn_mfma_prologue_kernel");
  // the score wavefronts work on packed scores: four lanes per query head with at most four heads per kv head
  // (or group), two lanes per head with five to eight
  const bool pack4 = a.QH / a.KVH <= 4;
  static bool configured = false;
  if (!configured) {
#define MF_CFG(B, P, L) AKV_HIP(hipFuncSetAttribute((const void*)akv_attn_mfma_kernel<B, P>, hipFuncAttributeMaxDynamicSharedMemorySize, L))
    MF_CFG(4, 2, MF_LDS_BYTES); MF_CFG(4, 4, MF_LDS_BYTES);
    MF_CFG(3, 2, MF_LDS_BYTES); MF_CFG(3, 4, MF_LDS_BYTES);
    MF_CFG(2, 2, MF_LDS_BYTES_2BIT); MF_CFG(2, 4, MF_LDS_BYTES_2BIT);
#undef MF_CFG
    configured = true;
  }
#define MF_RUN(B, L) do { if (pack4) AKV_LAUNCH_TIMED((akv_attn_mfma_kernel<B, 4>), grid, MF_THREADS, L, stream, a, x); \
                         else AKV_LAUNCH_TIMED((akv_attn_mfma_kernel<B, 2>), grid, MF_THREADS, L, stream, a, x); } while (0)
  if (bits == 4) MF_RUN(4, MF_LDS_BYTES);
  else if (bits == 3) MF_RUN(3, MF_LDS_BYTES);
  else MF_RUN(2, MF_LDS_BYTES_2BIT);
#undef MF_RUN
  AKV_LAUNCH_CHECK("akv_attn_mfma_kernel");
  return AKV_OK;
}

// ==================================================================================
// tq35 rows on the same machinery
// ==================================================================================
// A tq35 row is four parts per token: A0 (64 codes of 3 bits), B0 (64 sign bits), A1 (64 codes of
// 2 bits), B1 (64 sign bits), plus two fp16 factors per group inside the row.  Spread to one code
// per nibble they are 256 "virtual coordinates" over ONE table of sixteen levels -- 0..7 the 3-bit
// codebook, 8..11 the 2-bit codebook, 12 / 13 the signs -1 / +1 -- so the byte-pair tables and
// both products of the kernel above serve unchanged:
//
//   scores   four accumulators per 16-token tile, one per part (lane group g supplies nibble dwords
//            2g and 2g+1 of the part, four MFMAs per part), combined per token as
//            n0 (A0 + r0 B0) + n1 (A1 + r1 B1); the query operand holds the four transformed copies of
//            the query (aither_kvcache/hybrid_quantizer.py:600-640) in the coordinate order the
//            spreading leaves.
//   values   an M-tile mixes two parts so that a lane owns a dword-aligned piece of the row.  Pass C:
//            rows 0-7 the eight 3-byte groups of A0, rows 8-15 the eight halfwords of A1; pass S: rows
//            0-7 the sign bytes of B0, rows 8-15 those of B1.  The weight operand of a pass carries both
//            of its parts' weights (p n0 and p n1, or p n0 r0 and p n1 r1): columns 4t + q hold the fp16
//            part of set t for query head q of the group of four, columns 8 + 4t + q the remainder, and
//            a lane keeps the results whose rows belong to its column's set.  The V table holds
//            fp16(alpha c) with one alpha per codebook; pass S builds its operand straight from the sign
//            bits (fp16 -1 and +1 differ in one bit), no table; 1 / alpha and kappa = sqrt(pi/2)/64 are
//            applied to the finished sums (on the score side kappa rides in the query copies).
//
// One workgroup = 8 wavefronts: 4 score + 4 value (two passes of 8 accumulator tiles need twice the
// registers of the uniform formats), four groups of four query heads at a time.
#include "akv_hybrid_layout.h"

#define HM_HEADS 4
#define HM_THREADS 512
#define HM_NORMX ((uint32_t)MF_LDS_BYTES)    // float32 factors of a chunk: [parity][head slot][K | V][tile][field][16 tokens]
#define HM_WBUF2 (HM_NORMX + 2u * HM_HEADS * 1024u)   // weight operand of the second value pass
#define HM_LDS_BYTES (MF_LDS_BYTES + 4 * HM_HEADS * 1024)
#define HM_BITS_TAG 35

// level v of the merged table; the sign levels carry `sign_mag`
__device__ __forceinline__ float hm_level(const float* __restrict__ table, int v, float sign_mag) {
  return v < 12 ? table[HYB_CEN0 + v] : v == 12 ? -sign_mag : v == 13 ? sign_mag : 0.f;
}

// coordinate (0..63 inside its part) of nibble (byte b, lo = low nibble) of nibble dword D of part X
// (0 = A0, 1 = B0, 2 = A1, 3 = B1)
__host__ __device__ constexpr int hm_coord(int X, int D, int b, int lo) {
  if (X == 0) return 8 * D + mf_kcoord<3>(0, b, lo);
  if (X == 2) return 8 * D + (b == 0 ? 2 : b == 1 ? 0 : b == 2 ? 6 : 4) + lo;   // mf_spread2: bytes (c2,c3) (c0,c1) (c6,c7) (c4,c5)
  return 8 * D + 6 - 2 * b + lo;                                                  // hm_spread1: nibble i <- bit i <- coordinate 7 - i
}

// value side, 2-bit lanes: code of M-tile n (byte n/2; odd n = low nibble) among the lane's eight; the
// nibbles are [c3 c1 c7 c5 c2 c0 c6 c4] from bit 0 up
__host__ __device__ constexpr int hm_vcoord2(int n) {
  constexpr int nib[8] = {3, 1, 7, 5, 2, 0, 6, 4};
  return nib[2 * (n >> 1) + ((n & 1) ? 0 : 1)];
}

// eight sign bits (coordinate k at bit 7 - k) -> nibbles 12 | bit, nibble i <- bit i
__device__ __forceinline__ uint32_t hm_spread1(uint32_t b) {
  uint32_t t = (b | (b << 12)) & 0x000F000Fu;
  t = (t | (t << 6)) & 0x03030303u;
  return ((t | (t << 3)) & 0x11111111u) | 0xCCCCCCCCu;
}

template <int QDT>
__global__ __launch_bounds__(256) void akv_hyb_mfma_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ table,
    float kappa, float qscale, int S, int QH, int KVH, const void* context_lens, int cl_itype,
    int block_size, int64_t max_blocks_per_seq, int32_t* prefix, uint4* __restrict__ qop,
    uint32_t* __restrict__ lut, uint32_t* __restrict__ status) {
  __shared__ float qv[4][4][64];     // [query head of the group][part][coordinate]
  __shared__ int32_t scratch[257];
  __shared__ float best_err[256];
  __shared__ float best_alpha[256];
  const int tid = threadIdx.x;
  const int nq = S * KVH;
  if ((int)blockIdx.x == nq) {
    if (tid == 0) status[0] = 0u;
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, scratch);
    return;
  }
  if ((int)blockIdx.x == nq + 1) {
    // tables of the merged sixteen levels, rebuilt only when the codebooks in the table change
    __shared__ int stale;
    __shared__ float alphas[2];
    if (tid == 0) stale = (lut[MF_W_MARK] != MF_MARK + (uint32_t)HM_BITS_TAG) ? 1 : 0;
    __syncthreads();
    if (tid < 12 && __float_as_uint(table[HYB_CEN0 + tid]) != lut[MF_W_TAG + tid]) stale = 1;
    __syncthreads();
    if (!stale) return;
    // V table: fp16(alpha0 c) for the 3-bit codebook, fp16(alpha1 c) for the 2-bit codebook, each alpha in
    // [1,2) minimising the largest relative rounding error of its levels; the signs are exactly -1 / +1
    // (kappa and 1 / alpha are applied to the sums at the end)
    float c[12];
    for (int v = 0; v < 12; ++v) c[v] = table[HYB_CEN0 + v];
    for (int set = 0; set < 2; ++set) {
      const int v0 = set ? 8 : 0, v1 = set ? 12 : 8;
      float berr = 1e30f, balpha = 1.f;
      for (int k = 0; k < MF_ALPHA_CANDIDATES / 256; ++k) {
        const float al = 1.f + (float)(tid * (MF_ALPHA_CANDIDATES / 256) + k) / (float)MF_ALPHA_CANDIDATES;
        float worst = 0.f;
        for (int v = v0; v < v1; ++v) {
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
        lut[MF_W_ALPHA + set] = __float_as_uint(best_alpha[0]);
        alphas[set] = best_alpha[0];
      }
    }
    __syncthreads();
    auto vlevel = [&](int v) { return v < 8 ? alphas[0] * c[v] : v < 12 ? alphas[1] * c[v] : v == 12 ? -1.f : v == 13 ? 1.f : 0.f; };
    const float c0 = hm_level(table, tid >> 4, 1.f), c1 = hm_level(table, tid & 15, 1.f);
    const __half k0 = __float2half_rn(c0), k1 = __float2half_rn(c1);
    lut[MF_W_KHI + tid] = (unsigned)__half_as_ushort(k0) | ((unsigned)__half_as_ushort(k1) << 16);
    const __half l0 = __float2half_rn(c0 - __half2float(k0)), l1 = __float2half_rn(c1 - __half2float(k1));
    lut[MF_W_KLO + tid] = (unsigned)__half_as_ushort(l0) | ((unsigned)__half_as_ushort(l1) << 16);
    const __half v0 = __float2half_rn(vlevel(tid >> 4)), v1 = __float2half_rn(vlevel(tid & 15));
    lut[MF_W_VHI + tid] = (unsigned)__half_as_ushort(v0) | ((unsigned)__half_as_ushort(v1) << 16);
    if (tid < 12) lut[MF_W_TAG + tid] = __float_as_uint(table[HYB_CEN0 + tid]);
    __threadfence();
    __syncthreads();
    if (tid == 0) lut[MF_W_MARK] = MF_MARK + (uint32_t)HM_BITS_TAG;
    return;
  }
  const int s = blockIdx.x / KVH, hv = blockIdx.x % KVH;
  const int lane = tid & 63, w = tid >> 6;
  {
    const int64_t off = s * qs_seq + (int64_t)(hv * 4 + w) * qs_head;
    const float q0 = akv_elem<QDT>::load(query, off + lane);
    const float q1 = akv_elem<QDT>::load(query, off + 64 + lane);
    qv[w][0][lane] = hyb_fwht64(q0 * table[HYB_HAD0 + lane], lane) * 0.125f * qscale;
    qv[w][1][lane] = hyb_fwht64(q0 * table[HYB_QJL0 + lane], lane) * 0.125f * kappa * qscale;
    qv[w][2][lane] = hyb_fwht64(q1 * table[HYB_HAD1 + lane], lane) * 0.125f * qscale;
    qv[w][3][lane] = hyb_fwht64(q1 * table[HYB_QJL1 + lane], lane) * 0.125f * kappa * qscale;
  }
  __syncthreads();
  // operand layout: [k-step n = 4 X + n4][lane (col, g)][e]: nibble dword 2g + n4/2 of part X, byte
  // 2(n4 % 2) + e/4, nibble e % 2 (0 = high); elements 2,3 and 6,7 repeat 0,1 and 4,5 (they face the lo
  // halves of the K table entries); columns [0,4) the fp16 rounding of the query copy, [8,12) its remainder
  for (int n = w; n < 16; n += 4) {
    const int X = n >> 2, n4 = n & 3;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int D = 2 * g + (n4 >> 1), b = 2 * (n4 & 1) + (e >> 2), lo = e & 1;
      const int coord = hm_coord(X, D, b, lo);
      float v = 0.f;
      if (col < 4) {
        v = __half2float(__float2half_rn(qv[col][X][coord]));
      } else if (col >= 8 && col < 12) {
        const float full = qv[col - 8][X][coord];
        v = full - __half2float(__float2half_rn(full));
      }
      hbits[e] = __half_as_ushort(__float2half_rn(v));
    }
    uint4 o;
    o.x = hbits[0] | (hbits[1] << 16); o.y = hbits[2] | (hbits[3] << 16);
    o.z = hbits[4] | (hbits[5] << 16); o.w = hbits[6] | (hbits[7] << 16);
    qop[((size_t)(s * KVH + hv) * 16 + n) * 64 + lane] = o;
  }
}

struct hm_kraw {        // score wavefront, one 32-token chunk: the lane's pieces of token l%16 of both tiles
  mf_u32x2 a0[2];       // 8 bytes holding 3-byte groups 2g, 2g+1 of A0
  uint32_t b0[2];       // dword holding sign bytes 2g, 2g+1 of B0
  uint32_t a1[2];       // halfwords 2g, 2g+1 of A1
  uint32_t b1[2];
  uint32_t n0, n1;      // lane < 32: the two factor dwords of token l's K row, else of token (l - 32)'s V row
};
struct hm_vraw {        // value wavefront: tokens 4g + i of both tiles
  uint32_t c[8];        // pass C dword (A0 group col / A1 halfword col - 8)
  uint32_t s[8];        // pass S dword (sign byte)
};

template <int ROLE>
__device__ __forceinline__ void hm_role_main(const akv_hyb_mfma_args& a, const int hs) {
  const int lane = threadIdx.x & 63;
  const int col = lane & 15, g = lane >> 4;
  const uint32_t lane4v = MF_TABB + (uint32_t)(lane & 31) * 4u;
  const uint32_t lane4k = (uint32_t)(lane & 31) * 8u;
  // exchange buffers as in the kernel above: weights (16 B per reader lane L) at entry 32 hs + L/8,
  // rescale factors (4 B per lane) at entries 32 hs + 8, 9, flags at entry 32 hs + 12
  auto pbx = [&](uint32_t L) { return MF_TABB + (32u * hs + (L >> 3)) * 256u + 128u + (L & 7u) * 16u; };
  auto wsx = [&](uint32_t L) { return HM_WBUF2 + (uint32_t)hs * 1024u + L * 16u; };   // pass S weights: [parity][head slot][lane]
  auto rsx = [&](uint32_t L) { return MF_TABB + (32u * hs + 8u + (L >> 5)) * 256u + 128u + (L & 31u) * 4u; };
  const uint32_t fl_addr = MF_TABB + (32u * hs + 12u) * 256u + 128u;
  uint32_t T = 0;

  // blocks of 16 tokens: a chunk is two blocks; blocks of 32: one block, its second tile 16 positions further in
  const bool bs32 = a.block_size == 32;
  const int bs = bs32 ? 32 : 16;
  const int G = gridDim.x;
  const int total = a.prefix[a.S];
  const int per = (total + G - 1) / G;
  const int g0 = blockIdx.x * per;
  const int g1 = min(total, g0 + per);

  int gcur = g0;
  while (gcur < g1) {
    const int s = akv_find_seq(a.prefix, a.S, gcur);
    const int sb0 = a.prefix[s], sb1 = a.prefix[s + 1];
    const int blk_lo = gcur - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    const int64_t ctx = akv_seq_tokens(a.context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
    const int t_end = (int)min((int64_t)blk_hi * bs, ctx);
    gcur = sb0 + blk_hi;
    const int nblk = blk_hi - blk_lo;
    const int nchunks = bs32 ? nblk : (nblk + 1) >> 1;

    for (int hbase = 0; hbase < a.KVH; hbase += HM_HEADS) {
      const int h = hbase + hs;
      if (h >= a.KVH || nchunks <= 0) continue;
      const int hd = h / a.hgroup;      // the kv head whose rows are read

      int pbwin = 0, win_c0 = 0;
      auto load_window = [&](int c0) {
        const int bi = min(blk_lo + (bs32 ? c0 : 2 * c0) + lane, blk_hi - 1);
        pbwin = (int)akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + bi), a.num_blocks);
        asm volatile("" : "+v"(pbwin));
        win_c0 = c0;
      };
      auto chunk_blocks = [&](int c_in, uint32_t& p0, uint32_t& p1) {
        const int c = min(c_in, nchunks - 1);
        const int w0 = bs32 ? c - win_c0 : 2 * (c - win_c0);
        const int w1 = (!bs32 && 2 * c + 1 < nblk) ? w0 + 1 : w0;
        p0 = (uint32_t)__builtin_amdgcn_readlane(pbwin, w0);
        p1 = (uint32_t)__builtin_amdgcn_readlane(pbwin, w1);
      };
      load_window(0);

      if constexpr (ROLE == 0) {
        // =========================== score wavefront ===========================
        half8 qb[16];
        {
          const uint4* qp = a.qop + ((size_t)(s * a.KVH + h) * 16) * 64 + lane;
#pragma unroll
          for (int st = 0; st < 16; ++st) {
            const uint4 u = qp[st * 64];
            qb[st] = mf_pack(u.x, u.y, u.z, u.w);
          }
        }
        float m_run = -INFINITY, l_run = 0.f;
        const uint32_t krow = (uint32_t)(hd * a.kps_head + col * a.kps_pos);
        const uint32_t offA0 = krow + (g == 0 ? 0u : g == 1 ? 4u : g == 2 ? 12u : 16u);
        const uint32_t offB0 = krow + 24u + 4u * (uint32_t)(g >> 1);
        const uint32_t offA1 = krow + 36u + 4u * (uint32_t)g;
        const uint32_t offB1 = krow + 52u + 4u * (uint32_t)(g >> 1);
        const uint32_t selA = (g & 1) ? 0x0c020304u : 0x0c000102u;    // big-endian 24-bit words of the two groups
        const uint32_t selB = (g & 1) ? 0x0c050607u : 0x0c030405u;
        const uint32_t hsh = 16u * (uint32_t)(g & 1);
        const int ntok = lane & 31;
        const bool nrm_is_v = lane >= 32;
        const uint8_t* nrm_base = nrm_is_v ? a.vc : a.kc;
        const uint32_t nrm_blk = (uint32_t)(nrm_is_v ? a.vps_blk : a.kps_blk);
        const int npos = bs32 ? ntok : (ntok & 15);          // position of token ntok inside its block
        const uint32_t nrm_off = (uint32_t)(nrm_is_v ? hd * a.vps_head + npos * a.vps_pos
                                                     : hd * a.kps_head + npos * a.kps_pos);
        const uint32_t ktile1 = bs32 ? 16u * (uint32_t)a.kps_pos : 0u;
        // factor exchange: writer lane (kind = l/32, tile = (l/16)%2, token l%16) field f; reader lane (col, g)
        // takes tokens 4g..4g+3 of a (kind, tile, field) with one 16-byte read
        const uint32_t nw_addr = HM_NORMX + (uint32_t)hs * 1024u + (uint32_t)(lane >> 4) * 256u + (uint32_t)(lane & 15) * 4u;
        const uint32_t nr_addr = HM_NORMX + (uint32_t)hs * 1024u + (uint32_t)g * 16u;
        auto load_chunk = [&](hm_kraw& r, int c) {
          uint32_t pb[2];
          chunk_blocks(c, pb[0], pb[1]);
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const unsigned char* kb = a.kc + mf_umul(pb[j], (uint32_t)a.kps_blk) + (j ? ktile1 : 0u);
            r.a0[j] = *(const mf_u32x2*)(kb + mf_here(offA0));
            r.b0[j] = *(const uint32_t*)(kb + mf_here(offB0));
            r.a1[j] = *(const uint32_t*)(kb + mf_here(offA1));
            r.b1[j] = *(const uint32_t*)(kb + mf_here(offB1));
          }
          const unsigned char* nb = nrm_base + mf_umul(ntok >= 16 ? pb[1] : pb[0], nrm_blk) + mf_here(nrm_off);
          r.n0 = *(const uint32_t*)(nb + 32);
          r.n1 = *(const uint32_t*)(nb + 60);
        };
        auto half_lo = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w & 0xffffu))); };
        auto half_hi = [](uint32_t w) { return __half2float(__ushort_as_half((unsigned short)(w >> 16))); };
        auto produce = [&](hm_kraw& r, int c, const uint32_t par) {
          *(mf_lds_u32*)(uintptr_t)(nw_addr + 4096u * par) = __float_as_uint(half_lo(r.n0));
          *(mf_lds_u32*)(uintptr_t)(nw_addr + 4096u * par + 64u) = __float_as_uint(half_hi(r.n0));
          *(mf_lds_u32*)(uintptr_t)(nw_addr + 4096u * par + 128u) = __float_as_uint(half_lo(r.n1));
          *(mf_lds_u32*)(uintptr_t)(nw_addr + 4096u * par + 192u) = __float_as_uint(half_hi(r.n1));
          // nibble dwords: step n = 8 j + 2 X + Dl
          uint32_t kw[16];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            kw[8 * j + 0] = mf_spread3(__builtin_amdgcn_perm(r.a0[j].y, r.a0[j].x, selA));
            kw[8 * j + 1] = mf_spread3(__builtin_amdgcn_perm(r.a0[j].y, r.a0[j].x, selB));
            const uint32_t s0 = r.b0[j] >> hsh;
            kw[8 * j + 2] = hm_spread1(s0 & 0xffu);
            kw[8 * j + 3] = hm_spread1((s0 >> 8) & 0xffu);
            kw[8 * j + 4] = mf_spread2(r.a1[j] & 0xffffu) | 0x88888888u;
            kw[8 * j + 5] = mf_spread2(r.a1[j] >> 16) | 0x88888888u;
            const uint32_t s1 = r.b1[j] >> hsh;
            kw[8 * j + 6] = hm_spread1(s1 & 0xffu);
            kw[8 * j + 7] = hm_spread1((s1 >> 8) & 0xffu);
          }
          mf_u32x2 w[3][4];
          float4v acc[2][4];
#pragma unroll
          for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int X = 0; X < 4; ++X) acc[j][X] = (float4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int b = 0; b < 4; ++b) w[n][b] = mf_lut2(lane4k, kw[n], MF_SEL(b));
#pragma unroll
          for (int n = 0; n < 16; ++n) {
            if (n + 2 < 16) {
#pragma unroll
              for (int b = 0; b < 4; ++b) w[(n + 2) % 3][b] = mf_lut2(lane4k, kw[n + 2], MF_SEL(b));
            }
            const int j = n >> 3, X = (n >> 1) & 3, st = 2 * (n & 7);
            acc[j][X] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                mf_pack(w[n % 3][0].x, w[n % 3][0].y, w[n % 3][1].x, w[n % 3][1].y), qb[st], acc[j][X], 0, 0, 0);
            acc[j][X] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                mf_pack(w[n % 3][2].x, w[n % 3][2].y, w[n % 3][3].x, w[n % 3][3].y), qb[st + 1], acc[j][X], 0, 0, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
          load_chunk(r, c + 2);
          __builtin_amdgcn_sched_barrier(0);
          float sv[8];
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            union { mf_u32x4 u; float f[4]; } kn0, kr0, kn1, kr1;
            const uint32_t base = nr_addr + 4096u * par + 256u * j;
            kn0.u = *(mf_lds_u128*)(uintptr_t)(base);
            kr0.u = *(mf_lds_u128*)(uintptr_t)(base + 64u);
            kn1.u = *(mf_lds_u128*)(uintptr_t)(base + 128u);
            kr1.u = *(mf_lds_u128*)(uintptr_t)(base + 192u);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float t0 = fmaf(kr0.f[i], acc[j][1][i], acc[j][0][i]);
              const float t1 = fmaf(kr1.f[i], acc[j][3][i], acc[j][2][i]);
              const float raw = fmaf(kn1.f[i], t1, kn0.f[i] * t0);
              sv[4 * j + i] = raw + mf_from_hi_cols(raw);
            }
          }
          // From here on the wavefront works on a PACKED copy of the scores: the group has four query heads, so only
          // columns 0..3 of a row of sixteen lanes hold scores, eight per lane.  Lane 4k + c takes the token pair k
          // (values 2k, 2k + 1) of head c: two exponentials, eight weight products and four float16 splits per lane
          // and chunk in place of eight, thirty-two and sixteen; every lane then writes its own pair straight into
          // the operand fragments of the value side.
          const int kb = col >> 2, c4 = col & 3;
          float ps[2];
#pragma unroll
          for (int jj = 0; jj < 2; ++jj)
            ps[jj] = mf_to_bank<3>(mf_to_bank<2>(mf_to_bank<1>(sv[jj], sv[2 + jj]), sv[4 + jj]), sv[6 + jj]);
          // value-side factors of the lane's token pair (tile kb / 2, tokens 4g + 2 (kb % 2) + {0, 1})
          union { mf_u32x2 u; float f[2]; } vn0, vr0, vn1, vr1;
          {
            const uint32_t base = nr_addr + 4096u * par + 512u + 256u * (uint32_t)(kb >> 1) + 8u * (uint32_t)(kb & 1);
            vn0.u = *(mf_lds_cu64*)(uintptr_t)(base);
            vr0.u = *(mf_lds_cu64*)(uintptr_t)(base + 64u);
            vn1.u = *(mf_lds_cu64*)(uintptr_t)(base + 128u);
            vr1.u = *(mf_lds_cu64*)(uintptr_t)(base + 192u);
          }
          if (c == nchunks - 1) {     // only the last chunk of a segment can hold masked tokens (whose rows may hold anything)
            const int tok0 = blk_lo * bs + 32 * c + 16 * (kb >> 1) + 4 * g + 2 * (kb & 1);
            const bool tile_ok = (kb >> 1) == 0 || bs32 || 2 * c + 1 < nblk;
#pragma unroll
            for (int jj = 0; jj < 2; ++jj)
              if (!(tile_ok && tok0 + jj < t_end)) { ps[jj] = -INFINITY; vn0.f[jj] = 0.f; vr0.f[jj] = 0.f; vn1.f[jj] = 0.f; vr1.f[jj] = 0.f; }
          }
          const float mx = mf_rows_max(mf_banks_max(fmaxf(ps[0], ps[1])));
          const float m_new = fmaxf(m_run, mx);
          const float resc = __builtin_amdgcn_exp2f(m_run - m_new);
          m_run = m_new;
          float pw[4][2];
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            const float p = __builtin_amdgcn_exp2f(ps[jj] - m_new);
            pw[0][jj] = p * vn0.f[jj];
            pw[1][jj] = pw[0][jj] * vr0.f[jj];
            pw[2][jj] = p * vn1.f[jj];
            pw[3][jj] = pw[2][jj] * vr1.f[jj];
            ps[jj] = p;
          }
          l_run = l_run * resc + (ps[0] + ps[1]);       // the lane's own pair; summed over the banks when the segment ends
          mf_wait_ge(fl_addr + 4u, c >= 2 ? T + (uint32_t)c - 1u : T, a.status, a.spin_limit);
          // weight operand of pass P (0 = C: sets A0, A1; 1 = S: sets B0, B1): column 4 t + c holds the fp16 part of
          // set t of query head c, column 8 + 4 t + c its remainder; column k of the tile is read by lane 16 g + k,
          // whose sixteen bytes are the token pairs 0..3: this lane supplies dword kb of each
#pragma unroll
          for (int X = 0; X < 4; ++X) {
            auto h2 = __builtin_amdgcn_cvt_pkrtz(pw[X][0], pw[X][1]);
            auto l2 = __builtin_amdgcn_cvt_pkrtz(pw[X][0] - (float)h2[0], pw[X][1] - (float)h2[1]);
            union { decltype(h2) h; uint32_t u; } hb, lb;
            hb.h = h2;
            lb.h = l2;
            const uint32_t L = (uint32_t)(16 * g + 4 * (X >> 1) + c4);
            const uint32_t base = ((X & 1) ? wsx(L) + 4096u * par : pbx(L) + MF_XBUF * par) + 4u * (uint32_t)kb;
            const uint32_t base8 = ((X & 1) ? wsx(L + 8u) + 4096u * par : pbx(L + 8u) + MF_XBUF * par) + 4u * (uint32_t)kb;
            *(mf_lds_u32*)(uintptr_t)base = hb.u;
            *(mf_lds_u32*)(uintptr_t)base8 = lb.u;
          }
          *(mf_lds_u32*)(uintptr_t)(rsx((uint32_t)lane) + MF_XBUF * par) = __float_as_uint(resc);
          mf_publish(fl_addr, T + (uint32_t)c + 1u);
        };

        hm_kraw ra, rb;
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(ra, 0);
        __builtin_amdgcn_sched_barrier(0);
        load_chunk(rb, 1);
        __builtin_amdgcn_sched_barrier(0);
        int c = 0;
        for (; c + 1 < nchunks; c += 2) {
          if (c - win_c0 >= MF_WIN) load_window(c);
          produce(ra, c, 0);
          produce(rb, c + 1, 1);
        }
        if (c < nchunks) produce(ra, c, 0);
        __builtin_amdgcn_s_waitcnt(MF_WAIT_VM0);
        T += (uint32_t)nchunks;
        float lsum = l_run;
        lsum = mf_banks_sum(mf_rows_sum(lsum));
        if (col < 4 && g == 0) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * 4 + col);
          a.part_ml[slot * 2] = m_run * 0.6931471805599453f;
          a.part_ml[slot * 2 + 1] = lsum;
        }
      } else {
        // =========================== value wavefront ===========================
        float4v oC[8], oS[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) { oC[j] = (float4v){0.f, 0.f, 0.f, 0.f}; oS[j] = (float4v){0.f, 0.f, 0.f, 0.f}; }
        const int m = col;
        const bool is3 = m < 8;
        const uint32_t vrow = (uint32_t)(hd * a.vps_head + 4 * g * a.vps_pos);
        const uint32_t offC = vrow + (is3 ? 4u * (uint32_t)((3 * m) >> 2) : 36u + 4u * (uint32_t)((m - 8) >> 1));
        const uint32_t offS = vrow + (is3 ? 24u + 4u * (uint32_t)(m >> 2) : 52u + 4u * (uint32_t)((m - 8) >> 2));
        // pass C pieces as one word: lanes [0,8) the big-endian 24-bit word of 3-byte group m (from the
        // aligned dword holding its first byte and, where it runs over, the neighbour lane's dword), lanes
        // [8,16) halfword m - 8 of A1
        const uint32_t o3 = (uint32_t)(3 * m) & 3u;
        const uint32_t selC = is3 ? (0x0c000000u | (o3 << 16) | ((o3 + 1u) << 8) | (o3 + 2u))
                                  : ((m & 1) ? 0x0c0c0302u : 0x0c0c0100u);
        // ... spread to one code per nibble by five (shift, mask) terms whose constants differ by lane class:
        // mf_spread3 for the 3-bit lanes; for the 2-bit lanes (shift 0, mask 0x3333) and (shift 14, mask
        // 0x33330000) do the whole job (nibbles [c3 c1 c7 c5 c2 c0 c6 c4] from bit 0 up) and the levels
        // 8..11 of the merged table are selected by the constant 8 in every nibble
        const uint32_t cm0 = is3 ? 0x7007u : 0x3333u, corc = is3 ? 0u : 0x88888888u;
        const uint32_t cs1 = is3 ? 1u : 14u, cm1 = is3 ? 0x70070u : 0x33330000u;
        const uint32_t cm2 = is3 ? 0x700700u : 0u, cm3 = is3 ? 0x07000000u : 0u, cm4 = is3 ? 0x70000000u : 0u;
        const uint32_t selS = 0x0c000c00u | ((4u + (uint32_t)(m & 3)) << 16) | (uint32_t)(m & 3);
        const uint32_t vtile1 = bs32 ? 16u * (uint32_t)a.vps_pos : 0u;
        auto load_chunk = [&](hm_vraw& r, int c) {
          uint32_t pb[2];
          chunk_blocks(c, pb[0], pb[1]);
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const unsigned char* vb = a.vc + mf_umul(pb[j], (uint32_t)a.vps_blk) + (j ? vtile1 : 0u);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const unsigned char* vr = vb + (uint32_t)(i * (int)a.vps_pos);
              r.c[4 * j + i] = *(const uint32_t*)(vr + mf_here(offC));
              r.s[4 * j + i] = *(const uint32_t*)(vr + mf_here(offS));
            }
          }
        };
        // both constants of (x & mask) | pattern live in registers: as literals they would split the
        // operation in two
        uint32_t sgn_mask = 0x80008000u, one_pair = 0x3C003C00u;
        asm volatile("" : "+v"(sgn_mask));
        asm volatile("" : "+s"(one_pair));
        struct hm_vx { uint32_t ce[4], co[4], sg[4]; };   // token pairs: bytes of (high | low) nibbles; sign bytes
        auto transcode = [&](const hm_vraw& r, hm_vx& x) {
          uint32_t xc[8];
#pragma unroll
          for (int t = 0; t < 8; ++t) {
            const uint32_t wa = r.c[t];
            const uint32_t na = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)wa, 0x101 /*row_shl:1*/, 0xf, 0xf, true);
            const uint32_t w = __builtin_amdgcn_perm(na, wa, selC);
            uint32_t v = (w & cm0) | corc;
            v = ((w << cs1) & cm1) | v;
            v = ((w << 2) & cm2) | v;
            v = ((w << 15) & cm3) | v;
            v = ((w << 7) & cm4) | v;
            xc[t] = v;
          }
#pragma unroll
          for (int p = 0; p < 4; ++p) {
            x.ce[p] = (xc[2 * p] & 0xF0F0F0F0u) | ((xc[2 * p + 1] >> 4) & 0x0F0F0F0Fu);
            x.co[p] = ((xc[2 * p] << 4) & 0xF0F0F0F0u) | (xc[2 * p + 1] & 0x0F0F0F0Fu);
            // the lane's sign byte of token 2p in bits [0,8), of token 2p + 1 in bits [16,24)
            x.sg[p] = __builtin_amdgcn_perm(r.s[2 * p + 1], r.s[2 * p], selS);
          }
        };
        hm_vraw r;
        load_chunk(r, 0);
        for (int c = 0; c < nchunks; ++c) {
          const uint32_t par = (uint32_t)(c & 1);
          if (c - win_c0 >= MF_WIN) load_window(c);
          hm_vx x;
          transcode(r, x);
          __builtin_amdgcn_sched_barrier(0);
          load_chunk(r, c + 1);
          __builtin_amdgcn_sched_barrier(0);
          uint32_t wv[8][4];
#pragma unroll
          for (int n = 0; n < 8; ++n)
#pragma unroll
            for (int p = 0; p < 4; ++p) wv[n][p] = mf_lut(lane4v, (n & 1) ? x.co[p] : x.ce[p], MF_SEL(n >> 1));
          mf_wait_ge(fl_addr, T + (uint32_t)c + 1u, a.status, a.spin_limit);
          union { half8 h; mf_u32x4 u; } cv, cs;
          cv.u = *(mf_lds_u128*)(uintptr_t)(pbx((uint32_t)lane) + MF_XBUF * par);
          cs.u = *(mf_lds_u128*)(uintptr_t)(wsx((uint32_t)lane) + 4096u * par);
          const float resc = __uint_as_float(*(mf_lds_cu32*)(uintptr_t)(rsx((uint32_t)(16 * g + (col & 3))) + MF_XBUF * par));
          mf_publish(fl_addr + 4u, T + (uint32_t)c + 1u);
          if (__builtin_amdgcn_ballot_w64(resc != 1.f) != 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
#pragma unroll
              for (int i = 0; i < 4; ++i) { oC[j][i] *= resc; oS[j][i] *= resc; }
          }
#pragma unroll
          for (int n = 0; n < 8; ++n)
            oC[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(wv[n][0], wv[n][1], wv[n][2], wv[n][3]), cv.h, oC[n], 0, 0, 0);
          // pass S needs no table: fp16 -1 and +1 differ in the sign bit only, so the operand of tile n
          // (coordinate n of the byte = bit 7 - n) is that bit moved to bits 15 / 31 over the pattern of 1.0
          // (a set bit reads as -1 here; the sign is turned back with kappa at the end)
#pragma unroll
          for (int n = 0; n < 8; ++n) {
#pragma unroll
            for (int p = 0; p < 4; ++p) wv[n][p] = ((x.sg[p] << (8 + n)) & sgn_mask) | one_pair;
            oS[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(wv[n][0], wv[n][1], wv[n][2], wv[n][3]), cs.h, oS[n], 0, 0, 0);
          }
        }
        __builtin_amdgcn_s_waitcnt(MF_WAIT_VM0);
        T += (uint32_t)nchunks;
        // columns k and k + 8 carry the two fp16 terms of one weight; lane (column 4 t + q, g) then holds
        // rows 4g + i of every tile for set t of query head q, and rows [0,8) belong to set 0 (A0 in pass
        // C, B0 in pass S), rows [8,16) to set 1 (A1, B1)
        const int t = col >> 2, q = col & 3;
        const float inv_alpha = 1.f / __uint_as_float(a.lut[MF_W_ALPHA + (t & 1)]);
#pragma unroll
        for (int j = 0; j < 8; ++j)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            oC[j][i] = (oC[j][i] + mf_from_hi_cols(oC[j][i])) * inv_alpha;
            oS[j][i] = (oS[j][i] + mf_from_hi_cols(oS[j][i])) * -a.kappa;
          }
        if (col < 8 && (g >= 2) == (t == 1)) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * 4 + q);
          float* dst = a.part_acc + slot * 256 + 128 * t + 32 * (g & 1);      // parts A_t | B_t, rows 4 (g & 1) + i
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            float v[8], u[8];
            if (t == 0) {
#pragma unroll
              for (int n = 0; n < 8; ++n) v[hm_coord(0, 0, n >> 1, n & 1)] = oC[n][i];
            } else {
#pragma unroll
              for (int n = 0; n < 8; ++n) v[hm_vcoord2(n)] = oC[n][i];
            }
#pragma unroll
            for (int n = 0; n < 8; ++n) u[n] = oS[n][i];
            *(float4*)(dst + 8 * i) = make_float4(v[0], v[1], v[2], v[3]);
            *(float4*)(dst + 8 * i + 4) = make_float4(v[4], v[5], v[6], v[7]);
            *(float4*)(dst + 64 + 8 * i) = make_float4(u[0], u[1], u[2], u[3]);
            *(float4*)(dst + 64 + 8 * i + 4) = make_float4(u[4], u[5], u[6], u[7]);
          }
        }
      }
    }
  }
}

__global__ __launch_bounds__(HM_THREADS) void akv_hyb_mfma_kernel(akv_hyb_mfma_args a) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  {
    // thread (entry e, half hf) writes 16 of the entry's 32 copies
    const int e = threadIdx.x >> 1, hf = threadIdx.x & 1;
    const uint32_t khi = a.lut[MF_W_KHI + e], klo = a.lut[MF_W_KLO + e], vhi = a.lut[MF_W_VHI + e];
    uint4* ka = (uint4*)(lds_raw + e * 256 + hf * 128);
    uint4* va = (uint4*)(lds_raw + MF_TABB + e * 256 + hf * 64);
#pragma unroll
    for (int i = 0; i < 8; ++i) ka[i] = make_uint4(khi, klo, khi, klo);
#pragma unroll
    for (int i = 0; i < 4; ++i) va[i] = make_uint4(vhi, vhi, vhi, vhi);
  }
  if (threadIdx.x < HM_HEADS) *(uint2*)(lds_raw + MF_TABB + (32u * threadIdx.x + 12u) * 256u + 128u) = make_uint2(0u, 0u);
  __syncthreads();
  if ((wave >> 2) == 0) hm_role_main<0>(a, wave & 3);
  else hm_role_main<1>(a, wave & 3);
}

size_t akv_hyb_mfma_extra_bytes(int S, int QH) {
  return akv_align256((size_t)S * ((QH + 3) / 4) * 16 * 64 * 16);
}

// rows are dword-aligned (the caller checks); groups of four query heads; blocks of 16 or 32 tokens
bool akv_hyb_mfma_applicable(int QH, int KVH, int block_size, const int64_t* strides6) {
  if (mfma_disabled()) return false;
  const int gqa = QH / KVH;
  if (gqa % 4 != 0 || (block_size != 16 && block_size != 32)) return false;
  for (int i = 0; i < 6; ++i)
    if (strides6[i] < 0 || strides6[i] >= ((int64_t)1 << 27)) return false;
  return true;
}

int akv_hyb_mfma_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* table, float kappa,
                     float scale, akv_hyb_mfma_args a, int block_size, int32_t* prefix, uint32_t* lut, void* extra_ws,
                     int grid, hipStream_t stream) {
  a.block_size = block_size;
  a.hgroup = (a.QH / a.KVH) / 4;
  a.KVH *= a.hgroup;
  a.lut = lut;
  a.qop = (const uint4*)extra_ws;
  a.prefix = prefix;
  a.spin_limit = g_spin_limit;
  const float qscale = scale * 1.4426950408889634f;
  a.kappa = kappa;
  const int pgrid = a.S * a.KVH + 2;
#define HM_PRO(DT) akv_hyb_mfma_prologue_kernel<DT><<<pgrid, 256, 0, stream>>>(query, qs_seq, qs_head, table, kappa, qscale, a.S, a.QH, a.KVH, a.context_lens, a.cl_itype, block_size, a.max_blocks_per_seq, prefix, (uint4*)a.qop, (uint32_t*)a.lut, a.status)
  if (q_dtype == AKV_F16) HM_PRO(AKV_F16); else if (q_dtype == AKV_BF16) HM_PRO(AKV_BF16); else HM_PRO(AKV_F32);
#undef HM_PRO
  AKV_LAUNCH_CHECK("akv_hyb_mfma_prologue_kernel");
  static bool configured = false;
  if (!configured) {
    AKV_HIP(hipFuncSetAttribute((const void*)akv_hyb_mfma_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, HM_LDS_BYTES));
    configured = true;
  }
  AKV_LAUNCH_TIMED(akv_hyb_mfma_kernel, grid, HM_THREADS, HM_LDS_BYTES, stream, a);
  AKV_LAUNCH_CHECK("akv_hyb_mfma_kernel");
  return AKV_OK;
}
