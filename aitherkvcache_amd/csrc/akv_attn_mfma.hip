// MFMA paged decode attention for the 4-bit cache at head_dim 128, block_size 16.
//
// One workgroup = 8 wavefronts, wavefront <-> kv head; tokens are taken 32 at a time (two
// physical blocks).  Everything is arranged so that no register ever has to be transposed:
//
//   scores   S^T[token, col] = sum_d Khat[token, d] * Qop[d, col]       v_mfma_f32_16x16x32_f16
//            A = Khat: lane (n = l%16, g = l/16) owns bytes [16g, 16g+16) of token n's code row
//            (one 16-byte load); k-step s uses its dword s = coordinates 32g + 8s + 0..7.
//            B = Qop: the rotated queries of the kv head's query heads, in the same coordinate
//            order, columns [0,8) = fp16 rounding of q', columns [8,16) = fp16 of the remainder
//            (so the product carries q' to ~22 bits at no extra MFMA).
//            Result: lane (col, g) holds tokens 4g..4g+3 of the tile for column col.
//   softmax  running max / sum per column; the weights p * |v| / alpha of a lane are exactly the
//            k-slice of the B operand of the next product (tokens 4g..4g+3 of both tiles), again
//            split hi / lo over columns [0,8) / [8,16).
//   values   O^T[coord, col] += sum_token Vhat[token, coord] * P[token, col]
//            A = Vhat^T: lane (m, g) loads dword m (coordinates 8m..8m+7) of its 8 tokens and
//            builds, for each of the 8 coordinates, the 8-token k-slice; M-tile j row m is
//            coordinate 8m + j.
//
// Dequantisation goes through a table in LDS indexed by a whole BYTE: entry (a<<4|b) is the
// fp16 pair (alpha c[a], alpha c[b]).  For K a byte holds two neighbouring coordinates of one
// token -- already a k-pair.  For V the k axis is the token axis, so bytes are first re-formed
// from the same nibble position of two neighbouring tokens (two bit-field inserts per 8 codes).
// The table is replicated 64 times (address = byte * 256 + lane * 4) so that lookups never
// conflict on an LDS bank.  alpha in [1,2) is chosen per codebook so that alpha*c is almost
// exactly representable in fp16 (the rounding of the 16 levels would otherwise be the largest
// error of the whole computation); it is divided out of the scores and of the weights.
#include "akv_attn_common.h"

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));

#define MF_WAVES 8
#define MF_LUT_COPIES 32                       // copies of each half of an entry (lane & 31)
#define MF_LUT_BYTES (256 * 256)               // entry e at e*256: [hi pair x 32][lo pair x 32]
#ifndef MF_KSPLIT
#define MF_KSPLIT 1                            // scores use hi + lo table halves (2 MFMA per k-step)
#endif
#define MF_ALPHA_CANDIDATES 65536

struct akv_mfma_extra {
  const uint32_t* lut;   // [2][256] fp16 pairs: hi = fp16(alpha c), lo = fp16(alpha c - hi); then the tag (workspace)
  const float* alpha;    // [1]                         (workspace)
  const uint4* qop;      // [S][KVH][4 k-steps x 2 halves][64 lanes] half8 as uint4 (workspace)
};

// ----------------------------------------------------------------------------------
// prologue: q' = Pi q in MFMA operand layout, block prefix, byte-pair table
// ----------------------------------------------------------------------------------
template <int QDT>
__global__ __launch_bounds__(256) void akv_attn_mfma_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ PiT,
    const float* __restrict__ centroids, int S, int QH, int KVH, const void* context_lens,
    int cl_itype, int block_size, int64_t max_blocks_per_seq, int32_t* prefix,
    uint4* __restrict__ qop, uint32_t* __restrict__ lut, float* __restrict__ alpha_out) {
  __shared__ __align__(16) float q_lds[128][8];   // [input coordinate][query head of the group], zero-padded
  __shared__ float qr_lds[8][128];
  __shared__ int32_t scratch[257];
  __shared__ float best_err[256];
  __shared__ float best_alpha[256];
  const int tid = threadIdx.x;
  const int nq = S * KVH;
  if ((int)blockIdx.x == nq) {
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, scratch);
    return;
  }
  if ((int)blockIdx.x == nq + 1) {
    // The table depends on the codebook only.  It is kept in the workspace together with the
    // centroids it was built from (lut[512..527]) and a marker (lut[528]); when they match, the
    // search is skipped.
    __shared__ int stale;
    if (tid == 0) stale = (lut[528] != 0x7451u) ? 1 : 0;
    __syncthreads();
    if (tid < 16 && __float_as_uint(centroids[tid]) != lut[512 + tid]) stale = 1;
    __syncthreads();
    if (!stale) return;
    // alpha search: minimise the largest relative fp16 rounding error of alpha * c over the levels
    float c[16];
    for (int v = 0; v < 16; ++v) c[v] = centroids[v];
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
      alpha_out[0] = best_alpha[0];
    }
    __syncthreads();
    const float al = best_alpha[0];
    const float x0 = al * centroids[tid >> 4], x1 = al * centroids[tid & 15];   // pair (first, second)
    const __half h0 = __float2half_rn(x0), h1 = __float2half_rn(x1);
    lut[tid] = (unsigned)__half_as_ushort(h0) | ((unsigned)__half_as_ushort(h1) << 16);
    const __half l0 = __float2half_rn(x0 - __half2float(h0)), l1 = __float2half_rn(x1 - __half2float(h1));
    lut[256 + tid] = (unsigned)__half_as_ushort(l0) | ((unsigned)__half_as_ushort(l1) << 16);
    if (tid < 16) lut[512 + tid] = __float_as_uint(centroids[tid]);
    __threadfence();
    __syncthreads();
    if (tid == 0) lut[528] = 0x7451u;
    return;
  }
  const int s = blockIdx.x / KVH, h = blockIdx.x % KVH;
  const int gqa = QH / KVH;
  for (int i = tid; i < 8 * 128; i += 256) {
    const int q = i >> 7, j = i & 127;
    q_lds[j][q] = q < gqa ? akv_elem<QDT>::load(query, s * qs_seq + (h * gqa + q) * qs_head + j) : 0.f;
  }
  __syncthreads();
  {
    // thread (dim, half): partial dot products over 64 of the 128 input coordinates for every
    // query head of the group; the 64 matrix loads of a thread are independent and unrolled
    const int dim = tid & 127, half = tid >> 7;
    float part[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) part[q] = 0.f;
#pragma unroll 16
    for (int jj = 0; jj < 64; ++jj) {
      const int j = half * 64 + jj;
      const float pv = PiT[j * 128 + dim];
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
      for (int q = 0; q < 8; ++q) qr_lds[q][dim] += part[q];
    }
  }
  __syncthreads();
  // operand layout: [k-step st][half u][lane (col, g)][e].  The K operand of (st, u) holds, for
  // bytes 2u and 2u+1 of dword st of the lane's 16 code bytes, the hi pair then the lo pair of
  // the table entry: elements (0,1) hi / (2,3) lo of byte 2u, (4,5) hi / (6,7) lo of byte 2u+1.
  // So element e of the query operand is coordinate 32g + 8st + 4u + 2(e/4) + (e&1).
  for (int idx = tid; idx < 8 * 64; idx += 256) {
    const int su = idx >> 6, lane = idx & 63;
    const int st = su >> 1, u = su & 1;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int dim = 32 * g + 8 * st + 4 * u + 2 * (e >> 2) + (e & 1);
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
    qop[((size_t)(s * KVH + h) * 8 + su) * 64 + lane] = o;
  }
}

// ----------------------------------------------------------------------------------
// main kernel
// ----------------------------------------------------------------------------------
struct mf_raw {      // what one wavefront loads for one 32-token chunk
  uint4 k[2];        // K code rows: tile j, token l%16, bytes [16g, 16g+16)
  uint32_t v[8];     // V codes: token tau(g,e), dword l%16
  float kn[8], vn[8];  // norms of tokens 4g+i of tile 0 (i<4) and tile 1
};

typedef __attribute__((address_space(3))) const uint32_t mf_lds_u32;

// The table is the kernel's only LDS object, so it starts at LDS address 0 and a table address
// can be used as the LDS address itself (saves one add per lookup).
__device__ __forceinline__ uint32_t mf_lut(const unsigned char*, uint32_t lane4, uint32_t word, uint32_t sel) {
  // address = byte(word, k) * 256 + lane * 4, built by one byte permute:
  // result byte 0 <- lane4 byte 0 (selector 0x00), byte 1 <- word byte k (selector 0x04 + k), rest zero
  const uint32_t addr = __builtin_amdgcn_perm(word, lane4, sel);
  return *(mf_lds_u32*)(uintptr_t)addr;
}

// hi and lo halves of an entry in one go (the two loads differ by 128 bytes -> ds_read2_b32)
__device__ __forceinline__ void mf_lut2(const unsigned char*, uint32_t lane4, uint32_t word, uint32_t sel,
                                        uint32_t& hi, uint32_t& lo) {
  const uint32_t addr = __builtin_amdgcn_perm(word, lane4, sel);
  hi = *(mf_lds_u32*)(uintptr_t)addr;
  lo = *(mf_lds_u32*)(uintptr_t)(addr + 128);
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

__global__ __launch_bounds__(512) void akv_attn_mfma4_kernel(akv_attn_args a, akv_mfma_extra x) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wavefront-uniform on purpose
  const int col = lane & 15, g = lane >> 4;
  // replicate the table: dword index i = entry * 64 + half * 32 + copy
  {
    uint32_t* l32 = (uint32_t*)lds_raw;
    for (int i = threadIdx.x; i < 256 * 64; i += 512) l32[i] = x.lut[((i >> 5) & 1) * 256 + (i >> 6)];
  }
  const unsigned char* lut_lane = lds_raw;
  const uint32_t lane4 = (uint32_t)(lane & 31) * 4u;
  const float alpha = x.alpha[0];
  const float inv_alpha = 1.f / alpha;
  __syncthreads();

  const int G = gridDim.x;
  const int total = a.prefix[a.S];
  const int per = (total + G - 1) / G;
  const int g0 = blockIdx.x * per;
  const int g1 = min(total, g0 + per);
  const int gqa = a.QH / a.KVH;
  const float sc_mul = a.scale * inv_alpha;

  int gcur = g0;
  while (gcur < g1) {
    const int s = akv_find_seq(a.prefix, a.S, gcur);
    const int sb0 = a.prefix[s], sb1 = a.prefix[s + 1];
    const int blk_lo = gcur - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    const int64_t ctx = akv_seq_tokens(a.context_lens, a.cl_itype, s, 16, a.max_blocks_per_seq);
    const int t_end = (int)min((int64_t)blk_hi * 16, ctx);
    gcur = sb0 + blk_hi;
    const int nblk = blk_hi - blk_lo;
    const int nchunks = (nblk + 1) >> 1;

    for (int h = wave; h < a.KVH; h += MF_WAVES) {
      // query operand of this (sequence, kv head)
      half8 qb[8];
      {
        const uint4* qp = x.qop + ((size_t)(s * a.KVH + h) * 8) * 64 + lane;
#pragma unroll
        for (int su = 0; su < 8; ++su) {
          const uint4 u = qp[su * 64];
          qb[su] = mf_pack(u.x, u.y, u.z, u.w);
        }
      }
      float4v o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (float4v){0.f, 0.f, 0.f, 0.f};
      float m_run = -INFINITY, l_run = 0.f;

      // per-lane byte offsets inside a physical block (32-bit), added to a wavefront-uniform base
      const uint32_t koff = (uint32_t)(h * a.kps_head + col * a.kps_pos + 16 * g);
      uint32_t voff[4], knoff[4], vnoff[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        voff[i] = (uint32_t)(h * a.vps_head + (4 * g + i) * a.vps_pos + 4 * col);
        knoff[i] = (uint32_t)((h * a.kns_head + (4 * g + i) * a.kns_pos) * 4);
        vnoff[i] = (uint32_t)((h * a.vns_head + (4 * g + i) * a.vns_pos) * 4);
      }

      // physical block ids of the segment: lane i holds the id of block (window start + i); the
      // window is refreshed every 64 blocks, so the chunk loop itself reads no table entry
      // (a table load in the loop would make every prefetch wait for all loads before it)
      int pbwin = 0;
      auto load_window = [&](int first_blk) {
        const int bi = min(first_blk + lane, blk_hi - 1);
        pbwin = (int)akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + bi);
      };
      auto load_chunk = [&](mf_raw& r, int c) {
        if ((c & 31) == 0) load_window(blk_lo + 2 * c);
        const int w0 = (2 * c) & 63;
        const int w1 = (2 * c + 1 < nblk) ? w0 + 1 : w0;
        int64_t pb[2];
        pb[0] = __builtin_amdgcn_readlane(pbwin, w0);
        pb[1] = __builtin_amdgcn_readlane(pbwin, w1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const unsigned char* kb = a.kp + pb[j] * a.kps_blk;
          const unsigned char* vb = a.vp + pb[j] * a.vps_blk;
          const unsigned char* knb = (const unsigned char*)(a.kn + pb[j] * a.kns_blk);
          const unsigned char* vnb = (const unsigned char*)(a.vn + pb[j] * a.vns_blk);
          r.k[j] = *(const uint4*)(kb + koff);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            r.v[4 * j + i] = *(const uint32_t*)(vb + voff[i]);
            r.kn[4 * j + i] = *(const float*)(knb + knoff[i]);
            r.vn[4 * j + i] = *(const float*)(vnb + vnoff[i]);
          }
        }
      };

      auto process = [&](const mf_raw& r, int c) {
        const int tok0 = (blk_lo + 2 * c) * 16;      // first token of tile 0
        // ---- scores
        float sv[8];
        {
          // 16 steps (tile j, dword st, half u); the table reads of step n+1 are issued before
          // the MFMA of step n
          const uint32_t kw[8] = {r.k[0].x, r.k[0].y, r.k[0].z, r.k[0].w, r.k[1].x, r.k[1].y, r.k[1].z, r.k[1].w};
          uint32_t w[2][4];
          float4v acc[2];
          acc[0] = (float4v){0.f, 0.f, 0.f, 0.f};
          acc[1] = (float4v){0.f, 0.f, 0.f, 0.f};
          mf_lut2(lut_lane, lane4, kw[0], 0x0c0c0400u, w[0][0], w[0][1]);
          mf_lut2(lut_lane, lane4, kw[0], 0x0c0c0500u, w[0][2], w[0][3]);
#pragma unroll
          for (int n = 0; n < 16; ++n) {
            if (n + 1 < 16) {
              const int n1 = n + 1;
              const uint32_t word = kw[n1 >> 1];
              const uint32_t sel = 0x0c0c0400u + ((uint32_t)(2 * (n1 & 1)) << 8);
              mf_lut2(lut_lane, lane4, word, sel, w[n1 & 1][0], w[n1 & 1][1]);
              mf_lut2(lut_lane, lane4, word, sel + 0x100u, w[n1 & 1][2], w[n1 & 1][3]);
            }
            acc[n >> 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(w[n & 1][0], w[n & 1][1], w[n & 1][2], w[n & 1][3]),
                                                                 qb[n & 7], acc[n >> 3], 0, 0, 0);
          }
#pragma unroll
          for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              // columns c and c + 8 carry the hi and lo part of the same query head: both lanes form
              // the same sum, so the softmax state below is identical in the two
              // (both cross-lane moves run with all lanes active; only the choice is per lane)
              const float from_hi = mf_from_hi_cols(acc[j][i]);
              const float from_lo = mf_from_lo_cols(acc[j][i]);
              const float full = acc[j][i] + (col < 8 ? from_hi : from_lo);
              const int tok = tok0 + 16 * j + 4 * g + i;
              const bool ok = (tok < t_end) && (j == 0 || 2 * c + 1 < nblk);
              sv[4 * j + i] = ok ? full * r.kn[4 * j + i] * sc_mul : -INFINITY;
            }
          }
        }
        // ---- running softmax (per column; rows of 16 lanes hold different tokens)
        float mx = sv[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) mx = fmaxf(mx, sv[i]);
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
          const float resc = __expf(m_run - m_new);   // 0 on the first chunk (m_run = -inf)
          l_run *= resc;
#pragma unroll
          for (int j = 0; j < 8; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) o[j][i] *= resc;
          m_run = m_new;
        }
        // weights: hi part in columns [0,8), remainder in columns [8,16)
        half8 pb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __expf(sv[i] - m_run);      // exp(-inf) = 0 for masked tokens
          l_run += p;
          const float pw = p * r.vn[i] * inv_alpha;
          const float hi = __half2float(__float2half_rn(pw));
          pb[i] = (_Float16)(col < 8 ? hi : pw - hi);
        }
        // ---- values: pairs of tokens (2p, 2p+1) of this lane's eight -> bytes of (even | odd) coordinates
        uint32_t xe[4], xo[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const uint32_t wa = r.v[2 * p], wb = r.v[2 * p + 1];
          xe[p] = (wa & 0xF0F0F0F0u) | ((wb >> 4) & 0x0F0F0F0Fu);
          xo[p] = ((wa << 4) & 0xF0F0F0F0u) | (wb & 0x0F0F0F0Fu);
        }
        {
          // 8 steps: step n -> byte n/2 of the dword, even (xe) or odd (xo) coordinate; M-tile n
          uint32_t w[2][4];
#pragma unroll
          for (int p = 0; p < 4; ++p) w[0][p] = mf_lut(lut_lane, lane4, xe[p], 0x0c0c0400u);
#pragma unroll
          for (int n = 0; n < 8; ++n) {
            if (n + 1 < 8) {
              const int n1 = n + 1;
              const uint32_t sel = 0x0c0c0400u + ((uint32_t)(n1 >> 1) << 8);
#pragma unroll
              for (int p = 0; p < 4; ++p) w[n1 & 1][p] = mf_lut(lut_lane, lane4, (n1 & 1) ? xo[p] : xe[p], sel);
            }
            o[n] = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(w[n & 1][0], w[n & 1][1], w[n & 1][2], w[n & 1][3]),
                                                          pb, o[n], 0, 0, 0);
          }
        }
      };

      mf_raw ra, rb;
      if (nchunks > 0) load_chunk(ra, 0);
      for (int c = 0; c < nchunks; c += 2) {
        if (c + 1 < nchunks) load_chunk(rb, c + 1);
        process(ra, c);
        if (c + 1 < nchunks) {
          if (c + 2 < nchunks) load_chunk(ra, c + 2);
          process(rb, c + 1);
        }
      }

      // ---- partial: columns [0,8) + [8,16); lane (col < gqa, g) holds coordinates 32g + 8i + j
      float lsum = l_run;
      lsum += __shfl_xor(lsum, 16, 64);
      lsum += __shfl_xor(lsum, 32, 64);
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) o[j][i] += mf_from_hi_cols(o[j][i]);
      if (col < gqa) {
        const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * gqa + col);
        float* dst = a.part_acc + slot * 128 + 32 * g;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          *(float4*)(dst + 8 * i) = make_float4(o[0][i], o[1][i], o[2][i], o[3][i]);
          *(float4*)(dst + 8 * i + 4) = make_float4(o[4][i], o[5][i], o[6][i], o[7][i]);
        }
        if (g == 0) { a.part_ml[slot * 2] = m_run; a.part_ml[slot * 2 + 1] = lsum; }
      }
    }
  }
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
  return akv_align256(2304) + akv_align256(4) + akv_align256((size_t)S * KVH * 8 * 64 * 16);
}

bool akv_attn_mfma_applicable(const akv_attn_args& a, int d, int bits) {
  if (mfma_disabled()) return false;
  if (d != 128 || bits != 4 || a.block_size != 16) return false;
  const int gqa = a.QH / a.KVH;
  if (gqa > 8) return false;
  if ((((uintptr_t)a.kp | (uintptr_t)a.kps_blk | (uintptr_t)a.kps_pos | (uintptr_t)a.kps_head) & 15) != 0) return false;
  return true;
}

template <int QDT>
static void launch_mfma_prologue(const void* query, int64_t qs_seq, int64_t qs_head, const float* PiT,
                                 const akv_attn_args& a, int32_t* prefix, const akv_mfma_extra& x,
                                 hipStream_t stream) {
  akv_attn_mfma_prologue_kernel<QDT><<<a.S * a.KVH + 2, 256, 0, stream>>>(
      query, qs_seq, qs_head, PiT, a.centroids, a.S, a.QH, a.KVH, a.context_lens, a.cl_itype, a.block_size,
      a.max_blocks_per_seq, prefix, (uint4*)x.qop, (uint32_t*)x.lut, (float*)x.alpha);
}

int akv_attn_mfma_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* PiT,
                      const akv_attn_args& a, int32_t* prefix, void* extra_ws, int grid, hipStream_t stream) {
  akv_mfma_extra x;
  char* p = (char*)extra_ws;
  x.lut = (const uint32_t*)p; p += akv_align256(2304);
  x.alpha = (const float*)p; p += akv_align256(4);
  x.qop = (const uint4*)p;
  if (q_dtype == AKV_F16) launch_mfma_prologue<AKV_F16>(query, qs_seq, qs_head, PiT, a, prefix, x, stream);
  else if (q_dtype == AKV_BF16) launch_mfma_prologue<AKV_BF16>(query, qs_seq, qs_head, PiT, a, prefix, x, stream);
  else launch_mfma_prologue<AKV_F32>(query, qs_seq, qs_head, PiT, a, prefix, x, stream);
  AKV_LAUNCH_CHECK("akv_attn_mfma_prologue_kernel");
  static bool configured = false;
  if (!configured) {
    AKV_HIP(hipFuncSetAttribute((const void*)akv_attn_mfma4_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                MF_LUT_BYTES));
    configured = true;
  }
  akv_profile_mark_begin(stream);
  akv_attn_mfma4_kernel<<<grid, 512, MF_LUT_BYTES, stream>>>(a, x);
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("akv_attn_mfma4_kernel");
  return AKV_OK;
}
