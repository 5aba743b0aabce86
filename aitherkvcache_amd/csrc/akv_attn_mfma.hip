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
#define MF_ALPHA_CANDIDATES 4096

struct akv_mfma_extra {
  const uint32_t* lut;   // [2][256] fp16 pairs: hi = fp16(alpha c), lo = fp16(alpha c - hi)  (workspace)
  const float* alpha;    // [1]                         (workspace)
  const uint4* qop;      // [S][KVH][4 k-steps][64 lanes] half8 as uint4 (workspace)
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
  __shared__ float q_lds[8][128];
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
    return;
  }
  const int s = blockIdx.x / KVH, h = blockIdx.x % KVH;
  const int gqa = QH / KVH;
  for (int i = tid; i < gqa * 128; i += 256)
    q_lds[i >> 7][i & 127] = akv_elem<QDT>::load(query, s * qs_seq + (h * gqa + (i >> 7)) * qs_head + (i & 127));
  __syncthreads();
  {
    const int dim = tid & 127;
    for (int q = tid >> 7; q < gqa; q += 2) {
      float acc = 0.f;
      for (int j = 0; j < 128; ++j) acc = fmaf(PiT[j * 128 + dim], q_lds[q][j], acc);
      qr_lds[q][dim] = acc;
    }
  }
  __syncthreads();
  // operand layout: [k-step st][lane (col, g)][e] = coordinate 32g + 8st + e of column col
  {
    const int st = tid >> 6, lane = tid & 63;
    const int col = lane & 15, g = lane >> 4;
    unsigned short hbits[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int dim = 32 * g + 8 * st + e;
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
    qop[((size_t)(s * KVH + h) * 4 + st) * 64 + lane] = o;
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

__device__ __forceinline__ uint32_t mf_lut(const unsigned char* lds, uint32_t lane4, uint32_t word, uint32_t sel) {
  // address = byte(word, k) * 256 + lane * 4, built by one byte permute:
  // result byte 0 <- lane4 byte 0 (selector 0x00), byte 1 <- word byte k (selector 0x04 + k), rest zero
  const uint32_t addr = __builtin_amdgcn_perm(word, lane4, sel);
  return *(const uint32_t*)(lds + addr);
}

// hi and lo halves of an entry in one go (the two loads differ by 128 bytes -> ds_read2_b32)
__device__ __forceinline__ void mf_lut2(const unsigned char* lds, uint32_t lane4, uint32_t word, uint32_t sel,
                                        uint32_t& hi, uint32_t& lo) {
  const uint32_t addr = __builtin_amdgcn_perm(word, lane4, sel);
  hi = *(const uint32_t*)(lds + addr);
  lo = *(const uint32_t*)(lds + addr + 128);
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
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
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
      half8 qb[4];
      {
        const uint4* qp = x.qop + ((size_t)(s * a.KVH + h) * 4) * 64 + lane;
#pragma unroll
        for (int st = 0; st < 4; ++st) {
          const uint4 u = qp[st * 64];
          qb[st] = mf_pack(u.x, u.y, u.z, u.w);
        }
      }
      float4v o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (float4v){0.f, 0.f, 0.f, 0.f};
      float m_run = -INFINITY, l_run = 0.f;

      const unsigned char* kbase = a.kp + (int64_t)h * a.kps_head + (int64_t)col * a.kps_pos + 16 * g;
      const unsigned char* vbase = a.vp + (int64_t)h * a.vps_head + 4 * col;
      const float* knb = a.kn + (int64_t)h * a.kns_head;
      const float* vnb = a.vn + (int64_t)h * a.vns_head;

      auto load_chunk = [&](mf_raw& r, int c) {
        const int bi0 = blk_lo + 2 * c;
        const int bi1 = min(bi0 + 1, blk_hi - 1);
        int64_t pb[2];
        pb[0] = akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + bi0);
        pb[1] = akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + bi1);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          r.k[j] = *(const uint4*)(kbase + pb[j] * a.kps_blk);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int pos = 4 * g + i;
            r.v[4 * j + i] = *(const uint32_t*)(vbase + pb[j] * a.vps_blk + (int64_t)pos * a.vps_pos);
            r.kn[4 * j + i] = knb[pb[j] * a.kns_blk + (int64_t)pos * a.kns_pos];
            r.vn[4 * j + i] = vnb[pb[j] * a.vns_blk + (int64_t)pos * a.vns_pos];
          }
        }
      };

      auto process = [&](const mf_raw& r, int c) {
        const int tok0 = (blk_lo + 2 * c) * 16;      // first token of tile 0
        // ---- scores
        float sv[8];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float4v acc = (float4v){0.f, 0.f, 0.f, 0.f};
          const uint32_t kw[4] = {r.k[j].x, r.k[j].y, r.k[j].z, r.k[j].w};
#pragma unroll
          for (int st = 0; st < 4; ++st) {
#if MF_KSPLIT
            uint32_t h[4], lw[4];
            mf_lut2(lut_lane, lane4, kw[st], 0x0c0c0400u, h[0], lw[0]);
            mf_lut2(lut_lane, lane4, kw[st], 0x0c0c0500u, h[1], lw[1]);
            mf_lut2(lut_lane, lane4, kw[st], 0x0c0c0600u, h[2], lw[2]);
            mf_lut2(lut_lane, lane4, kw[st], 0x0c0c0700u, h[3], lw[3]);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(h[0], h[1], h[2], h[3]), qb[st], acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(mf_pack(lw[0], lw[1], lw[2], lw[3]), qb[st], acc, 0, 0, 0);
#else
            const half8 ka = mf_pack(mf_lut(lut_lane, lane4, kw[st], 0x0c0c0400u), mf_lut(lut_lane, lane4, kw[st], 0x0c0c0500u),
                                     mf_lut(lut_lane, lane4, kw[st], 0x0c0c0600u), mf_lut(lut_lane, lane4, kw[st], 0x0c0c0700u));
            acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka, qb[st], acc, 0, 0, 0);
#endif
          }
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            // columns c and c + 8 carry the hi and lo part of the same query head: both lanes form
            // the same sum, so the softmax state below is identical in the two
            // (both cross-lane moves run with all lanes active; only the choice is per lane)
            const float from_hi = mf_from_hi_cols(acc[i]);
            const float from_lo = mf_from_lo_cols(acc[i]);
            const float full = acc[i] + (col < 8 ? from_hi : from_lo);
            const int tok = tok0 + 16 * j + 4 * g + i;
            const bool ok = (tok < t_end) && (j == 0 || 2 * c + 1 < nblk);
            sv[4 * j + i] = ok ? full * r.kn[4 * j + i] * sc_mul : -INFINITY;
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
        float pw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __expf(sv[i] - m_run);      // exp(-inf) = 0 for masked tokens
          l_run += p;
          pw[i] = p * r.vn[i] * inv_alpha;
        }
        // hi part in columns [0,8), remainder in columns [8,16)
        half8 pb;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float hi = __half2float(__float2half_rn(pw[i]));
          pb[i] = (_Float16)(col < 8 ? hi : pw[i] - hi);
        }
        // ---- values: pairs of tokens (2p, 2p+1) of this lane's eight -> bytes of (even | odd) coordinates
        uint32_t xe[4], xo[4];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const uint32_t wa = r.v[2 * p], wb = r.v[2 * p + 1];
          xe[p] = (wa & 0xF0F0F0F0u) | ((wb >> 4) & 0x0F0F0F0Fu);
          xo[p] = ((wa << 4) & 0xF0F0F0F0u) | (wb & 0x0F0F0F0Fu);
        }
#pragma unroll
        for (int bi = 0; bi < 4; ++bi) {               // byte bi of the dword: coordinates 8m + 2bi, 8m + 2bi + 1
          const uint32_t sel = 0x0c0c0400u + ((uint32_t)bi << 8);
          const half8 ve = mf_pack(mf_lut(lut_lane, lane4, xe[0], sel), mf_lut(lut_lane, lane4, xe[1], sel),
                                   mf_lut(lut_lane, lane4, xe[2], sel), mf_lut(lut_lane, lane4, xe[3], sel));
          o[2 * bi] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ve, pb, o[2 * bi], 0, 0, 0);
          const half8 vo = mf_pack(mf_lut(lut_lane, lane4, xo[0], sel), mf_lut(lut_lane, lane4, xo[1], sel),
                                   mf_lut(lut_lane, lane4, xo[2], sel), mf_lut(lut_lane, lane4, xo[3], sel));
          o[2 * bi + 1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vo, pb, o[2 * bi + 1], 0, 0, 0);
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
  return akv_align256(2048) + akv_align256(4) + akv_align256((size_t)S * KVH * 4 * 64 * 16);
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
  x.lut = (const uint32_t*)p; p += akv_align256(2048);
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
