// TriAttention decode_step (aither_kvcache/triattention/attention.py:186-280 with
// TrigSeriesScorer.score, scorer.py:115-208).  Coefficients: int4 nibble pairs (the reference's default and the
// only width its paged cache stores), or -- in the general kernel only -- uint8 pairs / float16 pairs
// (scorer.py:84-113).  Post-RoPE scoring (scorer.py:200-202) is the same series at a position difference
// of zero: cos 0 = 1 and sin 0 = 0 exactly, which leaves sum_f c_f.
//
// Per (batch, kv head) the S cached tokens are cut into NSPLIT contiguous ranges, one
// wavefront each.  Lanes <-> tokens: a lane unpacks its token's F retained pairs, forms
//   c_f = q_e k0 + q_o k1,  s_f = q_o k0 - q_e k1   at the pair's index,
//   score = (1/sqrt(d)) sum_f (c_f cos(delta theta_f) + s_f sin(delta theta_f)),
// with delta = float(key_pos) - float(query_pos) and the phase formed by ONE float32 multiply
// as the reference does (phases reach ~3e4 rad, so the argument must match to the last bit
// before sin/cos).  The phases are shared by the GQ query heads of the kv head.  A running
// softmax is kept per wavefront.  The weighted sum of the sparse value rows is formed, at
// head_dim 128 (DENSE), on the matrix cores: the 64 tokens of a chunk scatter their retained
// coefficients into a dense [pair][token][even, odd] float16 tile in LDS (an int4 code c stands for
// (2c - 15)/15, and 2c - 15 is exact in float16), the softmax weights times the value scale go
// through LDS into the operand layout as float16 hi + lo, and sixteen v_mfma_f32_16x16x32_f16
// multiply them (rows = pairs, columns = (query head, even/odd, hi/lo), k = (token, even/odd) with
// zeros where the parities differ).  To keep the weights inside float16 the running maximum is
// taken over score + ln(value scale), so weight x scale <= 1.  Other head dims scatter-add into
// LDS bins with atomics.  A second kernel merges the NSPLIT partials with the log-sum-exp rule
// and writes float32.
#include "akv_common.h"

#define TRI_MAX_SPLITS 128
#define TRI_WAVES 4
// DENSE value tile of a wavefront: 64 pairs x (64 tokens x 4 bytes + 16 bytes of padding, so that the
// sixteen pairs read by one operand load fall into different banks), then the weight table
// [8 = hi/lo x 4 query heads] x (64 tokens x 2 bytes + 8)
#define TRI_VT_PITCH 272
#define TRI_WT_PITCH 136
#define TRI_VT_BYTES (64 * TRI_VT_PITCH)
#define TRI_DENSE_WAVE_BYTES (TRI_VT_BYTES + 8 * TRI_WT_PITCH)
#define TRI_WSCALE 16384.f          // weights are carried as float16 of (weight x scale) x 2^14

typedef _Float16 tri_half8 __attribute__((ext_vector_type(8)));
typedef _Float16 tri_half2 __attribute__((ext_vector_type(2)));
typedef float tri_float4 __attribute__((ext_vector_type(4)));

struct tri_args {
  const void* query; int q_dtype;
  const uint8_t* k_idx; const uint8_t* k_cf; const __half* k_sc;
  const uint8_t* v_idx; const uint8_t* v_cf; const __half* v_sc;
  const float* theta;
  const void* qpos; int qp_itype;
  const void* kpos; int kp_itype;
  int B; int64_t S; int QH, KVH, D, F;
  int cbits;       // coefficient width: 4 (a byte per pair), 8 (two bytes per pair), 16 (two float16 per pair, scales unused)
  int post_rope;   // keys were stored after RoPE: plain sparse dot product, positions unused
  int nsplit;
  int two_stages;      // all-heads kernel: the staging area exists twice and a step has one barrier instead of two
  // paged cache (arrays are [num_blocks][block_size][KVH][...]; S = max_blocks_per_seq * block_size)
  const void* block_tables; int bt_itype; int64_t bt_stride;
  const void* context_lens; int cl_itype;
  int block_size; int64_t num_blocks;
  // token -> block without a division: a shift when the block size is a power of two (bs_shift), else
  // floor(t / block_size) = (t x bs_magic) >> (32 + bs_mshift), exact for t < 2^30 and block sizes from 3
  int bs_shift; uint32_t bs_magic; int bs_mshift;
  float* part_acc;  // [B][QH][nsplit][D]
  float* part_ml;   // [B][QH][nsplit][2]
};

__device__ __forceinline__ float tri_dequant(uint32_t code, float scale) {
  // (code / 7.5 - 1) * scale, scorer.py:99-104
  return __fmul_rn(__fsub_rn(__fdiv_rn((float)code, 7.5f), 1.0f), scale);
}

// sin and cos of a float32 angle of any size reached by positions x frequencies (|x| < ~1e6), in
// revolutions: 1 / 2 pi = H + L with H the nearest float; k = rint(fl(x H)); the fused multiply-add
// x H - k is the exact product minus an integer, rounded once at the size of the remainder, and a second
// one adds x L.  The remainder is good to 6e-8 revolutions (checked against 80-bit arithmetic over 2e6
// arguments up to 1e6 rad; it can exceed 1/2 by the rounding of x H, which the hardware functions allow).
// The hardware sine and cosine take revolutions and are good to 1.3e-7 absolute on [-1/2, 1/2] (measured
// against double precision over 2^22 arguments).
__device__ __forceinline__ void tri_sincos(float x, float& sn, float& cs) {
  const float k = rintf(x * 0.15915493667125702f);
  float f = fmaf(x, 0.15915493667125702f, -k);
  f = fmaf(x, 6.4206382432985265e-09f, f);
  sn = __builtin_amdgcn_sinf(f);
  cs = __builtin_amdgcn_cosf(f);
}

// WIDE: the coefficient width is a.cbits (4, 8 or 16) instead of 4; only without F12
template <int GQ, bool F12, bool DENSE, bool WIDE>
__global__ __launch_bounds__(256) void tri_decode_kernel(tri_args a) {
  static_assert(!(F12 && WIDE), "rows of three dwords are the 4-bit layout");
  extern __shared__ __align__(16) unsigned char lds_raw[];
  constexpr int DQN = WIDE ? 256 : 16;
  float* theta = (float*)lds_raw;                         // [D/2]
  float* q_lds = theta + a.D / 2;                         // [GQ][D]   (per workgroup pass)
  float* dq = q_lds + GQ * a.D;                           // [DQN]: code / half - 1 with the reference's roundings
  float* acc_base = dq + DQN;                             // [TRI_WAVES][GQ][D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* acc = acc_base + (size_t)wave * GQ * a.D;
  // DENSE (head_dim 128): instead of bins updated by LDS atomics (which serialise when many tokens
  // retain the same pair -- the usual case), each wavefront has a 16-token x 128-coordinate tile
  // and a 64 x GQ weight table; a lane owns one coordinate pair and its sums stay in registers
  unsigned char* vt = (unsigned char*)acc_base + (size_t)wave * TRI_DENSE_WAVE_BYTES;
  unsigned char* wt = vt + TRI_VT_BYTES;
  if (DENSE) {   // every use leaves the tile zero again; weight rows of absent query heads stay zero
    for (int i = lane; i < TRI_DENSE_WAVE_BYTES / 4; i += 64) ((uint32_t*)vt)[i] = 0u;
  }
  // operand roles of the lane: column n = q + 4 e + 8 hl of the weight operand, row m of a 16-pair tile
  const int col_n = lane & 15, grp = lane >> 4;
  const int col_q = col_n & 3, col_e = (col_n >> 2) & 1;
  const uint32_t sel_lo = col_e ? 0x01000c0cu : 0x0c0c0100u;   // first token of a dword into the lane's parity slot
  const uint32_t sel_hi = col_e ? 0x03020c0cu : 0x0c0c0302u;   // second token
  const unsigned char* wt_rd = wt + (4 * (col_n >> 3) + col_q) * TRI_WT_PITCH + 8 * grp;
  const unsigned char* vt_rd = vt + col_n * TRI_VT_PITCH + 16 * grp;
  const int D = a.D, F = a.F;
  constexpr int FU = F12 ? 12 : 4;   // pair loops: all twelve steps unrolled (static register indices), else four
  const int gqa = a.QH / a.KVH;
  const int b = blockIdx.z, h = blockIdx.y;
  const int split = blockIdx.x * TRI_WAVES + wave;
  const float inv_sqrt_d = 1.0f / sqrtf((float)D);

  for (int i = threadIdx.x; i < D / 2; i += 256) theta[i] = a.theta[i];
  const int cb = WIDE ? a.cbits : 4;
  if ((int)threadIdx.x < DQN) dq[threadIdx.x] = __fsub_rn(__fdiv_rn((float)threadIdx.x, cb == 8 ? 127.5f : 7.5f), 1.0f);
  // DENSE: the value tile holds 2 code - (15 | 255) or the float16 values themselves
  const float vfac = cb == 4 ? 1.f / (15.f * TRI_WSCALE) : cb == 8 ? 1.f / (255.f * TRI_WSCALE) : 1.f / TRI_WSCALE;

  const int64_t per = (a.S + a.nsplit - 1) / a.nsplit;
  const int64_t s0 = min(a.S, (int64_t)split * per);
  const int64_t s1 = min(a.S, s0 + per);
  const float qp = a.qpos ? (float)akv_load_index(a.qpos, a.qp_itype, b) : (float)a.S;

  for (int qg = 0; qg < gqa; qg += GQ) {
    __syncthreads();
    for (int i = threadIdx.x; i < GQ * D; i += 256) {
      const int q = i / D, d = i % D;
      const int64_t off = ((int64_t)b * a.QH + (h * gqa + qg + q)) * D + d;
      const int slot = ((d >> 1) * GQ + q) * 2 + (d & 1);   // [pair][q][even, odd]: one pair index serves all GQ heads
      float v;
      if (a.q_dtype == AKV_F16) v = akv_elem<AKV_F16>::load(a.query, off);
      else if (a.q_dtype == AKV_BF16) v = akv_elem<AKV_BF16>::load(a.query, off);
      else v = akv_elem<AKV_F32>::load(a.query, off);
      q_lds[slot] = v;
    }
    if (!DENSE) {
      for (int i = lane; i < GQ * D; i += 64) acc[i] = 0.f;
    }
    __syncthreads();
    tri_float4 oacc[4];     // DENSE: pairs 16 mt + 4 grp + i of column col_n
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) oacc[mt] = (tri_float4){0.f, 0.f, 0.f, 0.f};

    float m[GQ], l[GQ];
#pragma unroll
    for (int q = 0; q < GQ; ++q) { m[q] = -INFINITY; l[q] = 0.f; }

    // One chunk of 64 tokens is fetched while the chunk before it is worked on: the token's position,
    // both scales and (F = 12, aligned arrays) its index and coefficient bytes as three dwords each.
    // Tokens past the end of the range re-read its last token (never out of bounds; S >= 1 here).
    // (Everything is kept as loaded -- raw halfwords, the position as two dwords -- and converted where
    // it is used, so that no load has to be waited for at the point of the fetch.)
    struct tri_raw { uint32_t ki[3], kc[3], vi[3], vc[3]; uint32_t kp_lo, kp_hi; unsigned short ksc, vsc; };
    const bool kp_wide = a.kpos && a.kp_itype == AKV_I64;
    const unsigned char* kp_base = a.kpos ? (const unsigned char*)a.kpos : (const unsigned char*)a.theta;
    auto fetch = [&](tri_raw& r, int64_t c0) {
      const int64_t tc = max((int64_t)0, min(c0 + lane, s1 - 1));
      const int64_t row = ((int64_t)b * a.S + tc) * a.KVH + h;
      // position: low dword, and the high dword of a 64-bit entry (the low one again otherwise); without
      // an array of positions the loads read the first frequency and the value is not used
      const int64_t pe = a.kpos ? ((int64_t)b * a.S + tc) * (kp_wide ? 8 : 4) : 0;
      r.kp_lo = *(const uint32_t*)(kp_base + pe);
      r.kp_hi = *(const uint32_t*)(kp_base + pe + (kp_wide ? 4 : 0));
      r.ksc = r.vsc = 0x3c00;                       // float16 pairs carry no scale: 1.0
      if (!WIDE || cb != 16) {
        r.ksc = ((const unsigned short*)a.k_sc)[row];
        r.vsc = ((const unsigned short*)a.v_sc)[row];
      }
      if (F12) {
        const uint32_t* p0 = (const uint32_t*)(a.k_idx + row * 12);
        const uint32_t* p1 = (const uint32_t*)(a.k_cf + row * 12);
        const uint32_t* p2 = (const uint32_t*)(a.v_idx + row * 12);
        const uint32_t* p3 = (const uint32_t*)(a.v_cf + row * 12);
#pragma unroll
        for (int w = 0; w < 3; ++w) { r.ki[w] = p0[w]; r.kc[w] = p1[w]; r.vi[w] = p2[w]; r.vc[w] = p3[w]; }
      }
    };
    tri_raw cur;
    fetch(cur, s0);
    for (int64_t c0 = s0; c0 < s1; c0 += 64) {
      const int64_t t = c0 + lane;
      const bool valid = t < s1;
      const int64_t tc = valid ? t : s1 - 1;
      const int64_t row = ((int64_t)b * a.S + tc) * a.KVH + h;
      tri_raw nxt;
      fetch(nxt, c0 + 64);
      const float kp = !a.kpos ? (float)tc
                       : kp_wide ? (float)(int64_t)(((uint64_t)cur.kp_hi << 32) | cur.kp_lo) : (float)(int32_t)cur.kp_lo;
      const float delta = a.post_rope ? 0.f : __fsub_rn(kp, qp);
      const float ksc = __half2float(__ushort_as_half(cur.ksc));
      float sc[GQ];
#pragma unroll
      for (int q = 0; q < GQ; ++q) sc[q] = 0.f;
#pragma unroll FU
      for (int f = 0; f < (F12 ? 12 : F); ++f) {
        const uint32_t idx = F12 ? (cur.ki[f >> 2] >> (8 * (f & 3))) & 255u : a.k_idx[row * F + f];
        float k0, k1;
        if (!WIDE || cb == 4) {
          const uint32_t cf = F12 ? (cur.kc[f >> 2] >> (8 * (f & 3))) & 255u : a.k_cf[row * F + f];
          k0 = __fmul_rn(dq[cf >> 4], ksc); k1 = __fmul_rn(dq[cf & 15u], ksc);
        } else if (cb == 8) {
          const uint8_t* pc = a.k_cf + (row * F + f) * 2;
          k0 = __fmul_rn(dq[pc[0]], ksc); k1 = __fmul_rn(dq[pc[1]], ksc);
        } else {
          const __half* pc = (const __half*)a.k_cf + (row * F + f) * 2;
          k0 = __half2float(pc[0]); k1 = __half2float(pc[1]);
        }
        const float ph = __fmul_rn(delta, theta[idx]);
        float sn, cs;
        tri_sincos(ph, sn, cs);
        // q_e (k0 cos - k1 sin) + q_o (k1 cos + k0 sin): the key pair is turned once for all query heads
        const float ka = k0 * cs - k1 * sn;
        const float kb = k1 * cs + k0 * sn;
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const float2 qq = *(const float2*)(q_lds + (idx * GQ + q) * 2);
          sc[q] = fmaf(qq.y, kb, fmaf(qq.x, ka, sc[q]));
        }
      }
      float p[GQ];
      bool rescale = false;
      float alpha[GQ];
      // DENSE: the value scale enters the running maximum, so that p x scale <= 1 (float16 operand)
      float vsc = 0.f, bias = 0.f;
      if (DENSE) {
        vsc = __half2float(__ushort_as_half(cur.vsc));
        bias = __logf(fmaxf(vsc, 5.9604645e-8f));
      }
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const float sv = valid ? sc[q] * inv_sqrt_d : -INFINITY;
        const float mn = fmaxf(m[q], akv_wave_max(sv + bias));
        alpha[q] = __expf(m[q] - mn);
        rescale |= (mn != m[q]);
        p[q] = valid ? __expf(sv - mn) : 0.f;
        l[q] = l[q] * alpha[q] + p[q];
        m[q] = mn;
      }
      if (DENSE) {
        if (rescale) {  // wavefront-uniform: m is the same in every lane
          float asel = alpha[0];
          if (GQ == 4) asel = col_q == 1 ? alpha[1 % GQ] : col_q == 2 ? alpha[2 % GQ] : col_q == 3 ? alpha[3 % GQ] : asel;
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) oacc[mt] *= asel;
        }
        // weights: float16 hi (truncated) + lo of p x scale x 2^14, one halfword per (column, token)
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const float w = p[q] * vsc * TRI_WSCALE;
          auto h2 = __builtin_amdgcn_cvt_pkrtz(w, 0.f);
          auto l2 = __builtin_amdgcn_cvt_pkrtz(w - (float)h2[0], 0.f);
          union { decltype(h2) h; uint32_t u; } hb, lb;
          hb.h = h2; lb.h = l2;
          *(uint16_t*)(wt + q * TRI_WT_PITCH + 2 * lane) = (uint16_t)hb.u;
          *(uint16_t*)(wt + (4 + q) * TRI_WT_PITCH + 2 * lane) = (uint16_t)lb.u;
        }
        if (valid) {
#pragma unroll FU
          for (int f = 0; f < (F12 ? 12 : F); ++f) {
            const uint32_t idx = F12 ? (cur.vi[f >> 2] >> (8 * (f & 3))) & 255u : a.v_idx[row * F + f];
            union { uint32_t u; tri_half2 h; } cv;
            if (!WIDE || cb == 4) {
              const uint32_t cf = F12 ? (cur.vc[f >> 2] >> (8 * (f & 3))) & 255u : a.v_cf[row * F + f];
              // (2a - 15, 2b - 15) as a float16 pair: 0x6400 + n is float16(1024 + n), minus 1039 is exact
              cv.u = (((cf >> 4) | ((cf & 15u) << 16)) << 1) + 0x64006400u;
              cv.h = cv.h - (tri_half2){(_Float16)1039.f, (_Float16)1039.f};
            } else if (cb == 8) {
              const uint8_t* pc = a.v_cf + (row * F + f) * 2;   // (2a - 255, 2b - 255): integers below 2^11, exact
              cv.h = (tri_half2){(_Float16)(float)(2 * (int)pc[0] - 255), (_Float16)(float)(2 * (int)pc[1] - 255)};
            } else {
              const uint16_t* pc = (const uint16_t*)a.v_cf + (row * F + f) * 2;
              cv.u = (uint32_t)pc[0] | ((uint32_t)pc[1] << 16);
            }
            *(uint32_t*)(vt + (idx & 63u) * TRI_VT_PITCH + 4 * lane) = cv.u;
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {     // 16 tokens per step: k = 2 x token + parity
          const uint2 wr = *(const uint2*)(wt_rd + 32 * ks);
          union { uint32_t u[4]; tri_half8 h; } bw;
          bw.u[0] = __builtin_amdgcn_perm(wr.x, wr.x, sel_lo);
          bw.u[1] = __builtin_amdgcn_perm(wr.x, wr.x, sel_hi);
          bw.u[2] = __builtin_amdgcn_perm(wr.y, wr.y, sel_lo);
          bw.u[3] = __builtin_amdgcn_perm(wr.y, wr.y, sel_hi);
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) {
            union { uint4 u; tri_half8 h; } av;
            av.u = *(const uint4*)(vt_rd + mt * 16 * TRI_VT_PITCH + 64 * ks);
            oacc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av.h, bw.h, oacc[mt], 0, 0, 0);
          }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (valid) {
#pragma unroll FU
          for (int f = 0; f < (F12 ? 12 : F); ++f) {
            const uint32_t idx = F12 ? (cur.vi[f >> 2] >> (8 * (f & 3))) & 255u : a.v_idx[row * F + f];
            *(uint32_t*)(vt + (idx & 63u) * TRI_VT_PITCH + 4 * lane) = 0u;
          }
        }
      } else {
      if (rescale) {  // wavefront-uniform: m is the same in every lane
#pragma unroll
        for (int q = 0; q < GQ; ++q)
          for (int i = lane; i < D; i += 64) acc[q * D + i] *= alpha[q];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      if (valid) {
        const float vs = __half2float(__ushort_as_half(cur.vsc));
#pragma unroll FU
        for (int f = 0; f < (F12 ? 12 : F); ++f) {
          const uint32_t idx = F12 ? (cur.vi[f >> 2] >> (8 * (f & 3))) & 255u : a.v_idx[row * F + f];
          float v0, v1;
          if (!WIDE || cb == 4) {
            const uint32_t cf = F12 ? (cur.vc[f >> 2] >> (8 * (f & 3))) & 255u : a.v_cf[row * F + f];
            v0 = __fmul_rn(dq[cf >> 4], vs); v1 = __fmul_rn(dq[cf & 15u], vs);
          } else if (cb == 8) {
            const uint8_t* pc = a.v_cf + (row * F + f) * 2;
            v0 = __fmul_rn(dq[pc[0]], vs); v1 = __fmul_rn(dq[pc[1]], vs);
          } else {
            const __half* pc = (const __half*)a.v_cf + (row * F + f) * 2;
            v0 = __half2float(pc[0]); v1 = __half2float(pc[1]);
          }
#pragma unroll
          for (int q = 0; q < GQ; ++q) {
            atomicAdd(&acc[q * D + 2 * idx], p[q] * v0);
            atomicAdd(&acc[q * D + 2 * idx + 1], p[q] * v1);
          }
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      cur = nxt;
    }
    if (split < a.nsplit) {
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const size_t slot = ((size_t)b * a.QH + (h * gqa + qg + q)) * a.nsplit + split;
        const float lsum = akv_wave_sum(l[q]);
        if (DENSE) {
          // hi column + lo column (eight lanes to the right), then the lanes of column (q, parity) store
#pragma unroll
          for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const float hi = oacc[mt][i];
              const float lo = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(hi), 0x108 /*row_shl:8*/, 0xf, 0xf, true));
              if (col_n < 8 && col_q == q)
                a.part_acc[slot * D + 2 * (16 * mt + 4 * grp + i) + col_e] = (hi + lo) * vfac;
            }
        } else {
          for (int i = lane; i < D; i += 64) a.part_acc[slot * D + i] = acc[q * D + i];
        }
        if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
      }
    }
  }
}

// ----------------------------------------------------------------------------------
// TrigSeriesScorer.score alone (aither_kvcache/triattention/scorer.py:115-208): the logits [B][QH][S] as
// float32, for callers that add a mask or look at the scores themselves (TriAttention.forward with an
// attention mask, attention.py:148-166).  Lane = token, one pass per group of GQ query heads of the kv head;
// the arithmetic is that of tri_decode_kernel's score phase.
// ----------------------------------------------------------------------------------
template <int GQ>
__global__ __launch_bounds__(256) void tri_scores_kernel(tri_args a, float* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* theta = (float*)lds_raw;            // [D/2]
  float* q_lds = theta + a.D / 2;            // [D/2][GQ][even, odd]
  float* dq = q_lds + GQ * a.D;              // [256]: code / half - 1 with the reference's roundings
  const int D = a.D, F = a.F, cb = a.cbits;
  const int gqa = a.QH / a.KVH;
  const int b = blockIdx.z, h = blockIdx.y;
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const bool valid = t < a.S;
  const int64_t tc = valid ? t : a.S - 1;
  const float inv_sqrt_d = 1.0f / sqrtf((float)D);
  for (int i = threadIdx.x; i < D / 2; i += 256) theta[i] = a.theta[i];
  dq[threadIdx.x] = __fsub_rn(__fdiv_rn((float)threadIdx.x, cb == 8 ? 127.5f : 7.5f), 1.0f);
  const float qp = a.qpos ? (float)akv_load_index(a.qpos, a.qp_itype, b) : (float)a.S;
  const float kp = a.kpos ? (float)akv_load_index(a.kpos, a.kp_itype, (int64_t)b * a.S + tc) : (float)tc;
  const float delta = a.post_rope ? 0.f : __fsub_rn(kp, qp);
  const int64_t row = ((int64_t)b * a.S + tc) * a.KVH + h;
  const float ksc = cb == 16 ? 1.f : __half2float(a.k_sc[row]);
  for (int qg = 0; qg < gqa; qg += GQ) {
    __syncthreads();
    for (int i = threadIdx.x; i < GQ * D; i += 256) {
      const int q = i / D, d = i % D;
      const int64_t off = ((int64_t)b * a.QH + (h * gqa + qg + q)) * D + d;
      float v;
      if (a.q_dtype == AKV_F16) v = akv_elem<AKV_F16>::load(a.query, off);
      else if (a.q_dtype == AKV_BF16) v = akv_elem<AKV_BF16>::load(a.query, off);
      else v = akv_elem<AKV_F32>::load(a.query, off);
      q_lds[((d >> 1) * GQ + q) * 2 + (d & 1)] = v;
    }
    __syncthreads();
    float sc[GQ];
#pragma unroll
    for (int q = 0; q < GQ; ++q) sc[q] = 0.f;
    for (int f = 0; f < F; ++f) {
      const uint32_t idx = a.k_idx[row * F + f];
      float k0, k1;
      if (cb == 4) {
        const uint32_t cf = a.k_cf[row * F + f];
        k0 = __fmul_rn(dq[cf >> 4], ksc); k1 = __fmul_rn(dq[cf & 15u], ksc);
      } else if (cb == 8) {
        const uint8_t* pc = a.k_cf + (row * F + f) * 2;
        k0 = __fmul_rn(dq[pc[0]], ksc); k1 = __fmul_rn(dq[pc[1]], ksc);
      } else {
        const __half* pc = (const __half*)a.k_cf + (row * F + f) * 2;
        k0 = __half2float(pc[0]); k1 = __half2float(pc[1]);
      }
      float sn, cs;
      tri_sincos(__fmul_rn(delta, theta[idx]), sn, cs);
      const float ka = k0 * cs - k1 * sn;
      const float kb = k1 * cs + k0 * sn;
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const float2 qq = *(const float2*)(q_lds + (idx * GQ + q) * 2);
        sc[q] = fmaf(qq.y, kb, fmaf(qq.x, ka, sc[q]));
      }
    }
    if (valid) {
#pragma unroll
      for (int q = 0; q < GQ; ++q) out[((int64_t)b * a.QH + (h * gqa + qg + q)) * a.S + t] = sc[q] * inv_sqrt_d;
    }
  }
}

// ----------------------------------------------------------------------------------
// head_dim 128, F = 12, up to 8 kv heads: one workgroup takes a token range for ALL kv heads
// ----------------------------------------------------------------------------------
// In the cache a token's rows of the kv heads lie side by side (12 bytes each), so a wavefront that
// follows one head reads 12 bytes out of every 12 x kv_heads and touches a cache line per lane.
// Here wavefront h still works on head h, but the chunk of 64 tokens x kv_heads rows is fetched by
// the whole workgroup as the contiguous run of bytes it is (thread i <-> row i: one dwordx3 load per
// array covers 768 contiguous bytes per wavefront), one chunk ahead, and passes through LDS:
// [array][head][token] entries of 16 bytes -- the row's 12 bytes and, in the fourth dword of the
// index entries, the row's scale -- written and read by one 16-byte LDS operation each (a head's
// tokens lie 32 bytes apart from the next head's, which spreads the writes of a token's heads over
// the banks).  Two workgroup barriers per chunk
// (staging written -> read, read -> overwritten).  The dense value tile takes 32 tokens at a time.
#define TRH_Q_PAD 16                // a pair's row of the query table: GQ x (even, odd) floats + 16 bytes, so that
                                    // rows start at sixteen different bank positions (eight without)
#define TRH_HEAD_PITCH (64 * 16 + 32)
#define TRH_VT_PITCH 144            // 32 tokens x 4 bytes + 16
#define TRH_VT_BYTES (64 * TRH_VT_PITCH)
#define TRH_WT_PITCH (64 * 4 + 64)    // [4 query heads] x (64 tokens x (hi, lo) + 64: heads 16 banks apart)
#define TRH_WAVE_BYTES (TRH_VT_BYTES + 4 * TRH_WT_PITCH)

__device__ __forceinline__ float tri_row16_max(float v) {
  // maximum over the lane's row of 16 by row rotations folded into the maximum instruction itself
  // (data-parallel primitives, no LDS crossbar; scores are never NaN-quieted on the way)
  asm("s_nop 1\n\t"      // a lane-crossing read needs two idle cycles after the register was written
      "v_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
      "s_nop 1\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf"
      : "+v"(v));
  return v;
}
// the same for four values at once: the four chains alternate, so no instruction reads the result of the
// one before it and the idle cycles are not needed after the first
__device__ __forceinline__ void tri_row16_max4(float& a, float& b, float& c, float& d) {
  asm("s_nop 1\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %2, %2, %2 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %3, %3, %3 row_ror:8 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %2, %2, %2 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %3, %3, %3 row_ror:4 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %2, %2, %2 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %3, %3, %3 row_ror:2 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %0, %0, %0 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %1, %1, %1 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %2, %2, %2 row_ror:1 row_mask:0xf bank_mask:0xf\n\t"
      "v_max_f32_dpp %3, %3, %3 row_ror:1 row_mask:0xf bank_mask:0xf"
      : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}
__device__ __forceinline__ float tri_rows_max(float v) {
  // the four rows: v_permlane32_swap / v_permlane16_swap fed the same value twice leave
  // (rows 0,1,0,1 | 2,3,2,3) and (rows 0,0,2,2 | 1,1,3,3)
  auto x = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(x[0]), __uint_as_float(x[1]));
  auto y = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(y[0]), __uint_as_float(y[1]));
}
__device__ __forceinline__ float tri_wave_max(float v) {
  v = tri_row16_max(v);
  // the four rows: v_permlane32_swap / v_permlane16_swap fed the same value twice leave
  // (rows 0,1,0,1 | 2,3,2,3) and (rows 0,0,2,2 | 1,1,3,3)
  auto x = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(x[0]), __uint_as_float(x[1]));
  auto y = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(y[0]), __uint_as_float(y[1]));
}

// PAGED: the arrays are a block pool, batch element b reads its tokens through row b of the block
// table up to its own context length (SpectralKVCache.fetch_sequence,
// aither_kvcache/triattention/cache.py:163-198, fused into the load; a chunk of 64 tokens is then
// four runs of contiguous bytes instead of one); key positions are 0..ctx-1, query_pos defaults to ctx.
typedef __attribute__((address_space(3))) const float tri_lds_cfloat;
typedef float tri_f32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) const tri_f32x2 tri_lds_cfloat2;

// Two wavefronts per kv head.  The SCORE wavefront of head h (wavefront h) forms the scores of a chunk of 64
// tokens (lane = token), keeps the running softmax and leaves the weights (x value scale, float16 hi + lo)
// and the factors by which earlier sums shrink in LDS; the VALUE wavefront (wavefront KVH + h) scatters the
// chunk's value coefficients into its dense tile and, one chunk behind, multiplies them by those weights on
// the matrix cores.  The workgroup barriers that order the staging area also order the hand-over
// (weights are double-buffered).  Four wavefronts share a SIMD instead of two: the chains of dependent
// LDS reads, transcendentals and products of one role run in the shadow of the other's.
#define TRR_WAVE_BYTES (TRH_VT_BYTES + 2 * 4 * TRH_WT_PITCH)
#define TRR_ALPHA_FLOATS 8          // per (buffer, head): four factors, then a flag "some factor differs from one"

// bytes of one pair's row of the query table: float16 queries are kept as they are (GQ x (even, odd) halves; the
// multiply-adds take them directly), others as float32 with 16 bytes of padding
static constexpr int tri_qrow_bytes(int gqa_pass, bool q_half) { return q_half ? gqa_pass * 4 : gqa_pass * 8 + TRH_Q_PAD; }

// One staging area: per role (keys, values) the index rows with the scale (16 bytes per token) and the coefficient
// rows (12 bytes per token), head after head.
#define TRH_CF_PITCH (64 * 12 + 32)
static constexpr size_t tri_stage_bytes(int kvh) { return 2 * (size_t)kvh * (TRH_HEAD_PITCH + TRH_CF_PITCH); }
static size_t tri_roles_lds_bytes(int kvh, int gqa_pass, bool q_half, bool two_stages) {
  return 64 * sizeof(float) + (size_t)kvh * 64 * tri_qrow_bytes(gqa_pass, q_half) + 64 +
         (two_stages ? 2 : 1) * tri_stage_bytes(kvh) + (size_t)kvh * TRR_WAVE_BYTES +
         2 * (size_t)kvh * TRR_ALPHA_FLOATS * sizeof(float);
}
// With the staging area doubled a step needs one workgroup barrier (chunk k + 1 is written into the area that
// chunk k - 1 was read from, and every wavefront has passed the barrier of chunk k since it read that one);
// taken whenever the 160 KB of LDS hold it.
static bool tri_two_stages(int kvh, int gqa_pass, bool q_half) {
  return tri_roles_lds_bytes(kvh, gqa_pass, q_half, true) <= 160 * 1024;
}

typedef __attribute__((address_space(3))) const tri_half2 tri_lds_chalf2;
typedef uint32_t tri_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t tri_u32x3 __attribute__((ext_vector_type(3), aligned(4)));
typedef float tri_f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) const tri_u32x4 tri_lds_cu32x4;
typedef __attribute__((address_space(3))) const tri_f32x4 tri_lds_cf32x4;

template <int GQ, bool PAGED, bool QH16, bool KP, bool BSP2>
__global__ __launch_bounds__(1024) void tri_decode_heads_kernel(tri_args a) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  const int KVH = a.KVH;
  float* theta = (float*)lds_raw;                               // [64]
  float* q_lds = theta + 64;                                    // [KVH][64 pairs][GQ][even, odd]
  constexpr int QROW = tri_qrow_bytes(GQ, QH16);                // bytes of one pair's row of the query table
  unsigned char* stage = (unsigned char*)q_lds + (size_t)KVH * 64 * QROW + 64;   // one or two staging areas
  const uint32_t stage_bytes = (uint32_t)tri_stage_bytes(KVH);
  unsigned char* tiles = stage + (a.two_stages ? 2 : 1) * (size_t)stage_bytes;
  float* alpha_lds = (float*)(tiles + (size_t)KVH * TRR_WAVE_BYTES);             // [2][KVH][TRR_ALPHA_FLOATS]
  const int tid = threadIdx.x, lane = tid & 63, wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool value_role = wv >= KVH;                            // wavefront-uniform
  const int h = value_role ? wv - KVH : wv;
  unsigned char* vt = tiles + (size_t)h * TRR_WAVE_BYTES;
  unsigned char* wt0 = vt + TRH_VT_BYTES;                        // weight buffer i at wt0 + i * 4 * TRH_WT_PITCH
  const int col_n = lane & 15, grp = lane >> 4;
  const int col_q = col_n & 3, col_e = (col_n >> 2) & 1;
  // a weight dword is (hi | lo << 16) of one token: the lane takes its half into its parity slot
  const uint32_t sel_w = (col_n >> 3) ? (col_e ? 0x03020c0cu : 0x0c0c0302u) : (col_e ? 0x01000c0cu : 0x0c0c0100u);
  const unsigned char* vt_rd = vt + col_n * TRH_VT_PITCH + 16 * grp;
  const int gqa = a.QH / KVH;
  const int b = blockIdx.y, split = blockIdx.x;
  const float inv_sqrt_d = 1.0f / sqrtf(128.f);
  const float theta_mine = tid < 64 ? a.theta[tid] : 0.f;

  // tokens of this batch element; ranges start on multiples of 64 (PAGED: of the block size too)
  // (token numbers fit 32 bits: the host sends longer sequences elsewhere)
  const int S = PAGED ? (int)max((int64_t)0, min(akv_load_index(a.context_lens, a.cl_itype, b), a.S)) : (int)a.S;
  const int per_raw = (int)(((uint32_t)S + (uint32_t)a.nsplit - 1u) / (uint32_t)a.nsplit);
  const int per = PAGED ? ((per_raw + 63) & ~63) : per_raw;
  const int s0 = min(S, split * per);
  const int s1 = min(S, s0 + per);
  const float qp = a.qpos ? (float)akv_load_index(a.qpos, a.qp_itype, b) : (float)S;
  const bool kp_wide = KP && a.kp_itype == AKV_I64;          // KP: key positions are given (otherwise 0..S-1)

  // the thread's row of a chunk: token r / KVH, head r % KVH; the first KVH wavefronts fetch the key arrays,
  // the others the value arrays
  const int r = tid - (value_role ? KVH * 64 : 0);
  const int my_t = r / KVH, my_h = r - my_t * KVH;
  // (inside an area: [keys: index rows | coefficient rows][values: index rows | coefficient rows])
  const size_t arr_i = (size_t)KVH * TRH_HEAD_PITCH, arr_c = (size_t)KVH * TRH_CF_PITCH, role_b = arr_i + arr_c;
  unsigned char* st_wr = stage + (value_role ? role_b : 0) + (size_t)my_h * TRH_HEAD_PITCH + my_t * 16;
  unsigned char* st_wr_c = stage + (value_role ? role_b : 0) + arr_i + (size_t)my_h * TRH_CF_PITCH + my_t * 12;
  const unsigned char* st_rd = stage + (value_role ? role_b : 0) + (size_t)h * TRH_HEAD_PITCH + lane * 16;
  const unsigned char* st_rd_c = stage + (value_role ? role_b : 0) + arr_i + (size_t)h * TRH_CF_PITCH + lane * 12;
  // (score wavefront: the value scale of its token is the fourth dword of the value side's index entry)
  const unsigned char* st_rd_o = stage + (value_role ? 0 : role_b) + (size_t)h * TRH_HEAD_PITCH + lane * 16 + 12;
  // Not PAGED: the rows of batch element b start at a wavefront-uniform address and a row is named by a
  // 32-bit number (the host sends longer sequences to the other kernel).
  const int64_t row_b = PAGED ? 0 : (int64_t)b * a.S * KVH;
  const uint32_t last_rel = (uint32_t)max(s1, 1) * KVH - 1;
  const uint8_t* src_idx = (value_role ? a.v_idx : a.k_idx) + row_b * 12;
  const uint8_t* src_cf = (value_role ? a.v_cf : a.k_cf) + row_b * 12;
  const unsigned char* src_sc = (const unsigned char*)(value_role ? a.v_sc : a.k_sc) + row_b * 2;
  const unsigned char* kp_b = KP ? (const unsigned char*)a.kpos + (int64_t)b * a.S * (kp_wide ? 8 : 4) : nullptr;
  const int s1m = s1 - 1;

  struct tri_rows { uint32_t x[2][3]; unsigned short sc; uint32_t kp_lo, kp_hi; };
  // PAGED: the block table entry of the thread's token of a chunk, as two dwords (both index widths by the
  // same two loads: a load under a branch would make every later wait a wait for all loads)
  const bool bt_wide = PAGED && a.bt_itype == AKV_I64;
  const unsigned char* bt_b = PAGED ? (const unsigned char*)a.block_tables + (int64_t)b * a.bt_stride * (bt_wide ? 8 : 4) : nullptr;
  const uint32_t blk_last = BSP2 ? (uint32_t)max(s1m, 0) >> a.bs_shift : 0u;
  const uint32_t blk_rows = (uint32_t)a.block_size * (uint32_t)KVH;
  const uint32_t row_in_blk = ((uint32_t)(s0 + my_t) & (uint32_t)(a.block_size - 1)) * (uint32_t)KVH + (uint32_t)my_h;
  uint32_t bt_lo = 0, bt_hi = 0;
  auto table_entry = [&](int c0) {
    uint32_t blk;
    if constexpr (BSP2) {
      blk = min((uint32_t)(c0 + my_t) >> a.bs_shift, blk_last);         // tokens past the range: its last block
    } else {
      const uint32_t tcl = (uint32_t)max(0, min(c0 + my_t, s1m));
      blk = __umulhi(tcl, a.bs_magic) >> a.bs_mshift;
    }
    const uint32_t be = blk * (bt_wide ? 8u : 4u);
    bt_lo = *(const uint32_t*)(bt_b + (size_t)be);
    bt_hi = *(const uint32_t*)(bt_b + (size_t)be + (bt_wide ? 4 : 0));
  };
  auto fetch = [&](tri_rows& rr, int c0) {
    const uint32_t* p0;
    const uint32_t* p1;
    if (PAGED) {
      // The table entry of the thread's token was requested one chunk earlier: everything between the two
      // barriers of a step is waited for by all sixteen wavefronts, a dependent load there is paid per chunk.
      const bool hi_zero = !bt_wide || bt_hi == 0u;
      if constexpr (BSP2) {
        // Blocks of 1 .. 64 tokens (a power of two): chunks start on multiples of the block size, so the
        // token's place inside its block never changes and a row is (block x rows per block + a constant);
        // 32-bit byte offsets from wavefront-uniform bases (the host sends larger caches to the other form).
        // An entry outside the cache belongs to a token past the range: any row of the cache serves.
        const uint32_t phys = hi_zero ? min(bt_lo, (uint32_t)a.num_blocks - 1u) : 0u;
        const uint32_t row = __umul24(phys, blk_rows) + row_in_blk;
        const uint32_t o12 = (row << 3) + (row << 2);
        p0 = (const uint32_t*)(src_idx + (size_t)o12);
        p1 = (const uint32_t*)(src_cf + (size_t)o12);
        rr.sc = *(const unsigned short*)(src_sc + (size_t)(row << 1));
      } else {
        const uint32_t tcl = (uint32_t)max(0, min(c0 + my_t, s1m));     // tokens past the range: its last token
        const uint32_t blk = __umulhi(tcl, a.bs_magic) >> a.bs_mshift;
        const uint32_t off = tcl - blk * (uint32_t)a.block_size;
        int64_t phys = bt_wide ? (int64_t)(((uint64_t)bt_hi << 32) | bt_lo) : (int64_t)(int32_t)bt_lo;
        phys = max((int64_t)0, min(phys, a.num_blocks - 1));                 // (an empty sequence reads a padding entry)
        const uint32_t row = ((uint32_t)phys * (uint32_t)a.block_size + off) * (uint32_t)KVH + (uint32_t)my_h;
        p0 = (const uint32_t*)(src_idx + (size_t)row * 12);
        p1 = (const uint32_t*)(src_cf + (size_t)row * 12);
        rr.sc = *(const unsigned short*)(src_sc + (size_t)row * 2);
      }
    } else {
      const uint32_t rel = min((uint32_t)c0 * KVH + r, last_rel);            // rows past the range: its last row
      p0 = (const uint32_t*)(src_idx + (size_t)(rel * 12u));
      p1 = (const uint32_t*)(src_cf + (size_t)(rel * 12u));
      rr.sc = *(const unsigned short*)(src_sc + (size_t)(rel * 2u));
    }
#pragma unroll
    for (int w = 0; w < 3; ++w) { rr.x[0][w] = p0[w]; rr.x[1][w] = p1[w]; }
    // the score wavefront's own token positions (lane = token), as two dwords
    if constexpr (PAGED) table_entry(c0 + 64);
    rr.kp_lo = 0; rr.kp_hi = 0;
    if constexpr (KP) {
      const uint32_t pe = value_role ? 0u : (uint32_t)max(0, min(c0 + lane, s1m)) * (kp_wide ? 8u : 4u);
      rr.kp_lo = *(const uint32_t*)(kp_b + (size_t)pe);
      rr.kp_hi = *(const uint32_t*)(kp_b + (size_t)pe + (kp_wide ? 4 : 0));
    }
  };

  {
    // One workgroup serves GQ query heads of every kv head (grid z: which ones).  (A loop over the groups
    // inside the kernel would keep every value that only one role uses alive through the other role's
    // loop as well -- the loop's back edge joins the two -- and the kernel then needs more than its 128
    // registers; a reload from scratch memory is counted with the global loads, so waiting for it
    // waits for every row in flight.)
    const int qg = blockIdx.z * GQ;
    // The first chunk and the queries are requested before anything waits: the workgroup has KVH x 128
    // threads and KVH x GQ x 128 query elements, GQ per thread (element j of thread tid is number
    // tid + j x KVH x 128).
    tri_rows nxt;
    if constexpr (PAGED) table_entry(s0);
    fetch(nxt, s0);
    float qv[GQ];
    unsigned short qraw[GQ];
#pragma unroll
    for (int j = 0; j < GQ; ++j) {
      const int i = tid + j * KVH * 128;
      const int hh = i / (GQ * 128), rem = i - hh * (GQ * 128);
      const int q = rem >> 7, d = rem & 127;
      const int64_t off = ((int64_t)b * a.QH + (hh * gqa + qg + q)) * 128 + d;
      qv[j] = 0.f; qraw[j] = 0;
      if (QH16) qraw[j] = ((const unsigned short*)a.query)[off];
      else if (a.q_dtype == AKV_BF16) qv[j] = akv_elem<AKV_BF16>::load(a.query, off);
      else qv[j] = akv_elem<AKV_F32>::load(a.query, off);
    }
    {   // every use leaves a tile zero again; weight rows of absent query heads stay zero
      for (int i = tid; i < KVH * (TRR_WAVE_BYTES / 16); i += KVH * 128) ((uint4*)tiles)[i] = make_uint4(0u, 0u, 0u, 0u);
      if (tid < 64) theta[tid] = theta_mine;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < GQ; ++j) {
      const int i = tid + j * KVH * 128;
      const int hh = i / (GQ * 128), rem = i - hh * (GQ * 128);
      const int q = rem >> 7, d = rem & 127;
      unsigned char* row = (unsigned char*)q_lds + ((size_t)hh * 64 + (d >> 1)) * QROW;
      if (QH16) *(unsigned short*)(row + (q * 2 + (d & 1)) * 2) = qraw[j];
      else *(float*)(row + (q * 2 + (d & 1)) * 4) = qv[j];
    }
    const uint32_t q_base = 64 * sizeof(float) + (uint32_t)h * 64 * QROW;
    // One step of the staging pipeline, the same in both roles (two workgroup barriers): the chunk fetched
    // during the previous step goes to the staging area, the next one is requested, the wavefront's own
    // two entries per token come back.
    uint32_t kp_lo = 0, kp_hi = 0;
    uint32_t area = 0;                 // byte offset of the staging area of this step
    auto stage_step = [&](int c0, uint4& e0, tri_u32x3& e1, uint32_t& other_sc) {
      *(uint4*)(st_wr + area) = make_uint4(nxt.x[0][0], nxt.x[0][1], nxt.x[0][2], nxt.sc);
      *(tri_u32x3*)(st_wr_c + area) = (tri_u32x3){nxt.x[1][0], nxt.x[1][1], nxt.x[1][2]};
      kp_lo = nxt.kp_lo; kp_hi = nxt.kp_hi;
      __syncthreads();
      fetch(nxt, c0 + 64);
      e0 = *(const uint4*)(st_rd + area);
      e1 = *(const tri_u32x3*)(st_rd_c + area);
      other_sc = *(const uint32_t*)(st_rd_o + area);
      if (a.two_stages) area ^= stage_bytes;            // (wavefront-uniform)
      else __syncthreads();
    };

    if (!value_role) {
      float m[GQ], l[GQ];
#pragma unroll
      for (int q = 0; q < GQ; ++q) { m[q] = -INFINITY; l[q] = 0.f; }
      int buf = 0;
      for (int c0 = s0; c0 < s1; c0 += 64) {
        uint4 e0;
        tri_u32x3 e1;
        uint32_t vsc_raw;
        stage_step(c0, e0, e1, vsc_raw);
        const int t = c0 + lane;
        const bool valid = t < s1;
        const uint32_t ki[3] = {e0.x, e0.y, e0.z}, kc[3] = {e1.x, e1.y, e1.z};
        const float ksc = __half2float(__ushort_as_half((unsigned short)e0.w));
        const float vsc = __half2float(__ushort_as_half((unsigned short)vsc_raw));
        const float kp = !KP ? (float)(valid ? t : s1m)
                         : kp_wide ? (float)(int64_t)(((uint64_t)kp_hi << 32) | kp_lo) : (float)(int32_t)kp_lo;
        const float delta = a.post_rope ? 0.f : __fsub_rn(kp, qp);
        const float kscale = ksc * (inv_sqrt_d / 15.f);
        float sc[GQ];
#pragma unroll
        for (int q = 0; q < GQ; ++q) sc[q] = 0.f;
        // Per word of four pairs: the index bytes times 4 (a pair index is below 64, so the shift stays
        // inside its byte) and the two nibbles of every coefficient byte in bytes of their own; a byte
        // then becomes a float by one conversion.  A code c stands for (2c - 15)/15 x scale -- equal to
        // the reference's fl(fl(c/7.5) - 1) x scale to a relative 1e-7 -- and scale/15 multiplies the
        // finished sum instead of every coefficient.
        uint32_t ki4[3], chi[3], clo[3];
#pragma unroll
        for (int w = 0; w < 3; ++w) {
          ki4[w] = (ki[w] & 0x3f3f3f3fu) << 2;
          chi[w] = (kc[w] >> 4) & 0x0f0f0f0fu;
          clo[w] = kc[w] & 0x0f0f0f0fu;
          // (kept opaque: otherwise the masks are folded into one bit-field extract per code and the
          // conversion no longer selects its byte by itself)
          asm("" : "+v"(ki4[w]));
          asm("" : "+v"(chi[w]));
          asm("" : "+v"(clo[w]));
        }
#pragma unroll
        for (int f = 0; f < 12; ++f) {
          const uint32_t idx4 = (ki4[f >> 2] >> (8 * (f & 3))) & 255u;          // byte offset of theta[idx]
          const float k0 = fmaf((float)((chi[f >> 2] >> (8 * (f & 3))) & 255u), 2.f, -15.f);
          const float k1 = fmaf((float)((clo[f >> 2] >> (8 * (f & 3))) & 255u), 2.f, -15.f);
          // (the dynamic LDS of this kernel starts at LDS address 0 and theta is its first object: the
          // byte offset is the address, no base to add)
          const float ph = __fmul_rn(delta, *(tri_lds_cfloat*)(uintptr_t)idx4);
          float sn, cs;
          tri_sincos(ph, sn, cs);
          const float ka = k0 * cs - k1 * sn;
          const float kb = k1 * cs + k0 * sn;
          const uint32_t qrow = idx4 * (QROW / 4) + q_base;      // LDS address of the pair's row of this head
          if constexpr (GQ == 4 && QH16) {
            const tri_u32x4 qv = *(tri_lds_cu32x4*)(uintptr_t)qrow;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const uint32_t qw = qv[q];
              const tri_half2 qq = __builtin_bit_cast(tri_half2, qw);
              sc[q] = fmaf((float)qq.y, kb, fmaf((float)qq.x, ka, sc[q]));
            }
          } else if constexpr (GQ == 4) {
            const tri_f32x4 qa = *(tri_lds_cf32x4*)(uintptr_t)qrow;
            const tri_f32x4 qb = *(tri_lds_cf32x4*)(uintptr_t)(qrow + 16);
            sc[0] = fmaf(qa[1], kb, fmaf(qa[0], ka, sc[0]));
            sc[1] = fmaf(qa[3], kb, fmaf(qa[2], ka, sc[1]));
            sc[2] = fmaf(qb[1], kb, fmaf(qb[0], ka, sc[2]));
            sc[3] = fmaf(qb[3], kb, fmaf(qb[2], ka, sc[3]));
          } else {
#pragma unroll
            for (int q = 0; q < GQ; ++q) {
              if (QH16) {
                const tri_half2 qq = *(tri_lds_chalf2*)(uintptr_t)(qrow + 4 * q);
                sc[q] = fmaf((float)qq.y, kb, fmaf((float)qq.x, ka, sc[q]));
              } else {
                const tri_f32x2 qq = *(tri_lds_cfloat2*)(uintptr_t)(qrow + 8 * q);
                sc[q] = fmaf(qq.y, kb, fmaf(qq.x, ka, sc[q]));
              }
            }
          }
        }
        float p[GQ], alpha[GQ];
        // (the bias only places the maxima: the hardware logarithm is good enough, and a float16 scale is
        // never a float32 denormal)
        const float bias = __builtin_amdgcn_logf(fmaxf(vsc, 5.9604645e-8f)) * 0.6931471805599453f;
        float sv[GQ], mx[GQ];
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          sv[q] = valid ? sc[q] * kscale : -INFINITY;
          mx[q] = sv[q] + bias;
        }
        // The maxima are searched only when some token of the chunk exceeds one of them (the running
        // maxima are the same in every lane, so the test is one comparison per query head and a vote);
        // otherwise every factor is one and the sums just grow.
        float* al = alpha_lds + ((size_t)buf * KVH + h) * TRR_ALPHA_FLOATS;
        bool grow = false;
#pragma unroll
        for (int q = 0; q < GQ; ++q) grow |= mx[q] > m[q];
        if (__builtin_amdgcn_ballot_w64(grow) != 0ull) {
          if (GQ == 4) {
            tri_row16_max4(mx[0], mx[1 % GQ], mx[2 % GQ], mx[3 % GQ]);
#pragma unroll
            for (int q = 0; q < GQ; ++q) mx[q] = tri_rows_max(mx[q]);
          } else {
#pragma unroll
            for (int q = 0; q < GQ; ++q) mx[q] = tri_wave_max(mx[q]);
          }
#pragma unroll
          for (int q = 0; q < GQ; ++q) {
            const float mn = fmaxf(m[q], mx[q]);
            alpha[q] = __expf(m[q] - mn);
            l[q] *= alpha[q];
            m[q] = mn;
          }
          if (lane < 5) {        // m is the same in every lane, and so are the factors; entry 4: "some factor is not one"
            float av = 1.f;
#pragma unroll
            for (int q = 0; q < GQ; ++q) av = lane == q ? alpha[q] : av;
            if (lane < GQ || lane == 4) al[lane] = av;
          }
        } else if (lane == 4) {
          al[4] = 0.f;
        }
        // (a token past the range has the score minus infinity and the weight exp(-inf) = 0: the maxima
        // are finite once a chunk has been seen, and every chunk has a token inside the range)
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          p[q] = __expf(sv[q] - m[q]);
          l[q] += p[q];
        }
        // weight x value scale x 2^14 as float16 hi + lo: hi is the weight cut to float16's eleven bits, lo the
        // exact rest; one conversion packs the two
        unsigned char* wt = wt0 + buf * 4 * TRH_WT_PITCH;
        const float wsc = vsc * TRI_WSCALE;
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const float w = p[q] * wsc;
          const float w_hi = __uint_as_float(__float_as_uint(w) & 0xffffe000u);
          union { decltype(__builtin_amdgcn_cvt_pkrtz(0.f, 0.f)) hv; uint32_t u; } pk;
          pk.hv = __builtin_amdgcn_cvt_pkrtz(w_hi, w - w_hi);
          *(uint32_t*)(wt + q * TRH_WT_PITCH + 4 * lane) = pk.u;
        }
        buf ^= 1;
      }
      __syncthreads();             // (the value wavefronts wait here for the weights of the last chunk)
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const size_t slot = ((size_t)b * a.QH + (h * gqa + qg + q)) * a.nsplit + split;
        const float lsum = akv_wave_sum(l[q]);
        if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
      }
    } else {
      tri_float4 oacc[4];
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) oacc[mt] = (tri_float4){0.f, 0.f, 0.f, 0.f};
      // tile entries of the chunk whose weights are still being made
      uint32_t voff[12], vval[12];
      bool have_prev = false, prev_valid = false;
      // weights of buffer bufc times the tile entries kept in voff / vval
      auto consume = [&](int bufc) {
        const float* al = alpha_lds + ((size_t)bufc * KVH + h) * TRR_ALPHA_FLOATS;
        if (al[4] != 0.f) {      // wavefront-uniform
          const float asel = al[GQ == 4 ? col_q : 0];
#pragma unroll
          for (int mt = 0; mt < 4; ++mt) oacc[mt] *= asel;
        }
        const unsigned char* wt_rd = wt0 + bufc * 4 * TRH_WT_PITCH + col_q * TRH_WT_PITCH + 16 * grp;
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {      // the tile holds 32 tokens
          const bool mine = prev_valid && (lane >> 5) == pass;
          if (mine) {
#pragma unroll
            for (int f = 0; f < 12; ++f) *(uint32_t*)(vt + voff[f]) = vval[f];
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
          for (int ks = 0; ks < 2; ++ks) {
            const uint4 wr = *(const uint4*)(wt_rd + 64 * (2 * pass + ks));
            union { uint32_t u[4]; tri_half8 hv; } bw;
            bw.u[0] = __builtin_amdgcn_perm(wr.x, wr.x, sel_w);
            bw.u[1] = __builtin_amdgcn_perm(wr.y, wr.y, sel_w);
            bw.u[2] = __builtin_amdgcn_perm(wr.z, wr.z, sel_w);
            bw.u[3] = __builtin_amdgcn_perm(wr.w, wr.w, sel_w);
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
              union { uint4 u; tri_half8 hv; } av;
              av.u = *(const uint4*)(vt_rd + mt * 16 * TRH_VT_PITCH + 64 * ks);
              oacc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(av.hv, bw.hv, oacc[mt], 0, 0, 0);
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          if (mine) {
#pragma unroll
            for (int f = 0; f < 12; ++f) *(uint32_t*)(vt + voff[f]) = 0u;
          }
        }
      };
      int buf = 0;
      for (int c0 = s0; c0 < s1; c0 += 64) {
        uint4 e0;
        tri_u32x3 e1;
        uint32_t unused;
        stage_step(c0, e0, e1, unused);
        if (have_prev) consume(buf ^ 1);
        // tile entries of the lane's token: address and (2a - 15, 2b - 15) as a float16 pair, formed once
        // (0x6400 + n is float16(1024 + n); minus 1039 is exact)
        // (the nibbles of a word of four coefficient bytes in bytes of their own; one byte permute then
        // puts a pair's two codes into the low bytes of the two halves)
        const uint32_t vi[3] = {e0.x, e0.y, e0.z}, vc[3] = {e1.x, e1.y, e1.z};
        const uint32_t lane_off = 4 * (lane & 31);
#pragma unroll
        for (int f = 0; f < 12; ++f) {
          const uint32_t idx = (vi[f >> 2] >> (8 * (f & 3))) & 63u;
          const uint32_t hiw = (vc[f >> 2] >> 4) & 0x0f0f0f0fu, low = vc[f >> 2] & 0x0f0f0f0fu;
          const uint32_t pair = __builtin_amdgcn_perm(low, hiw, 0x0c040c00u + 0x00010001u * (f & 3));
          union { uint32_t u; tri_half2 hv; } cv;
          cv.u = (pair << 1) + 0x64006400u;
          cv.hv = cv.hv - (tri_half2){(_Float16)1039.f, (_Float16)1039.f};
          vval[f] = cv.u;
          voff[f] = idx * TRH_VT_PITCH + lane_off;
        }
        have_prev = true;
        prev_valid = c0 + lane < s1;
        buf ^= 1;
      }
      __syncthreads();             // the weights of the last chunk
      if (have_prev) consume(buf ^ 1);
      {
        // columns 0..7 hold the high parts of (query head, parity), columns 8..15 the low parts
        const size_t slot = ((size_t)b * a.QH + (h * gqa + qg + (GQ == 4 ? col_q : 0))) * a.nsplit + split;
        float* dst = a.part_acc + slot * 128 + 8 * grp + col_e;
        const bool mine = col_n < 8 && col_q < GQ;
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float hi = oacc[mt][i];
            const float lo = __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(hi), 0x108 /*row_shl:8*/, 0xf, 0xf, true));
            if (mine) dst[32 * mt + 2 * i] = (hi + lo) * (1.f / (15.f * TRI_WSCALE));
          }
      }
    }
  }
}

// one workgroup per (batch, query head): split weights once, then one thread per coordinate
__global__ __launch_bounds__(128) void tri_reduce_kernel(const float* __restrict__ part_acc,
                                                         const float* __restrict__ part_ml,
                                                         int nsplit, int D, float* __restrict__ out) {
  __shared__ float w[TRI_MAX_SPLITS];
  __shared__ float red[2];
  const size_t pair = blockIdx.x;  // b * QH + qh
  // the first partial sums of the thread's coordinate are requested before the weights exist: the
  // two round trips to memory overlap (D <= 128 coordinates take one pass of the 128 threads)
  constexpr int PRE = 32;
  float pre[PRE];
  {
    const int i0 = min((int)threadIdx.x, D - 1);
#pragma unroll
    for (int s = 0; s < PRE; ++s) pre[s] = part_acc[(pair * nsplit + min(s, nsplit - 1)) * D + i0];
  }
  if (threadIdx.x < 64) {
    // (maximum, sum) of ranges lane and lane + 64, one 8-byte load each, requested together
    static_assert(TRI_MAX_SPLITS <= 128, "two ranges per lane");
    const int sa = threadIdx.x, sb = threadIdx.x + 64;
    float2 mla = make_float2(-INFINITY, 0.f), mlb = make_float2(-INFINITY, 0.f);
    if (sa < nsplit) mla = *(const float2*)(part_ml + (pair * nsplit + sa) * 2);
    if (sb < nsplit) mlb = *(const float2*)(part_ml + (pair * nsplit + sb) * 2);
    const float m = akv_wave_max(fmaxf(mla.x, mlb.x));
    const float wa = mla.x > -INFINITY ? __expf(mla.x - m) : 0.f;
    const float wb = mlb.x > -INFINITY ? __expf(mlb.x - m) : 0.f;
    if (sa < nsplit) w[sa] = wa;
    if (sb < nsplit) w[sb] = wb;
    const float l = akv_wave_sum(wa * mla.y + wb * mlb.y);
    if (threadIdx.x == 0) red[0] = l > 0.f ? 1.f / l : 0.f;
  }
  __syncthreads();
  const float inv = red[0];
  // (every range writes its partial sums, zeros when it holds no token: the loads need no guard and
  // can all be in flight together)
  for (int i = threadIdx.x; i < D; i += 128) {
    float acc = 0.f;
    const float* src = part_acc + pair * nsplit * D + i;
    int s0 = 0;
    if (i == (int)threadIdx.x) {          // first pass: the prefetched ranges
#pragma unroll
      for (int s = 0; s < PRE; ++s) acc = fmaf(s < nsplit ? w[s] : 0.f, pre[s], acc);
      s0 = PRE;
    }
#pragma unroll 16
    for (int s = s0; s < nsplit; ++s) acc = fmaf(w[s], src[(size_t)s * D], acc);
    out[pair * D + i] = acc * inv;
  }
}

__global__ void tri_zero_kernel(float* out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = 0.f;
}

// launch of the all-heads kernel for (gq, qh, lds, hgrid, num_kv_heads, stream, a) of the caller; more than 64 KB
// of dynamic LDS has to be allowed once per kernel
template <int GQ, bool PAGED, bool QH16, bool KP, bool BSP2>
static int tri_heads_launch(dim3 hgrid, int kvh, size_t lds, hipStream_t stream, const tri_args& a) {
  static size_t configured = 0;
  if (configured < lds) {
    AKV_HIP(hipFuncSetAttribute((const void*)tri_decode_heads_kernel<GQ, PAGED, QH16, KP, BSP2>,
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    configured = lds;
  }
  AKV_LAUNCH_TIMED((tri_decode_heads_kernel<GQ, PAGED, QH16, KP, BSP2>), hgrid, kvh * 128, lds, stream, a);
  return AKV_OK;
}
#define TRI_HEADS_LAUNCH(PAGED, KP, BSP2)                                                                            \
  do {                                                                                                               \
    int rc_;                                                                                                         \
    if (gq == 4) rc_ = qh ? tri_heads_launch<4, PAGED, true, KP, BSP2>(hgrid, num_kv_heads, lds, stream, a)          \
                          : tri_heads_launch<4, PAGED, false, KP, BSP2>(hgrid, num_kv_heads, lds, stream, a);        \
    else rc_ = qh ? tri_heads_launch<1, PAGED, true, KP, BSP2>(hgrid, num_kv_heads, lds, stream, a)                  \
                  : tri_heads_launch<1, PAGED, false, KP, BSP2>(hgrid, num_kv_heads, lds, stream, a);                \
    if (rc_ != AKV_OK) return rc_;                                                                                   \
  } while (0)

static int tri_pick_splits(int batch, int kvh, int64_t S) {
  int cus = akv_cached_cu_count();
  if (cus <= 0) cus = 256;
  int64_t want = ((int64_t)cus * 16 + (int64_t)batch * kvh - 1) / ((int64_t)batch * kvh);
  int64_t by_len = (S + 63) / 64;
  int64_t n = want < by_len ? want : by_len;
  if (n < 1) n = 1;
  n = (n + TRI_WAVES - 1) / TRI_WAVES * TRI_WAVES;
  if (n > TRI_MAX_SPLITS) n = TRI_MAX_SPLITS;
  return (int)n;
}

extern "C" size_t akv_tri_decode_workspace_bytes(int batch, int num_q_heads, int d) {
  if (batch <= 0 || num_q_heads <= 0 || d <= 0) return 0;
  return (size_t)batch * num_q_heads * TRI_MAX_SPLITS * (d + 2) * sizeof(float) + 256;
}

extern "C" int akv_tri_decode_step(const void* query, int q_dtype, const uint8_t* k_indices,
                                   const void* k_coeffs, const void* k_scales,
                                   const uint8_t* v_indices, const void* v_coeffs,
                                   const void* v_scales, const float* theta, const void* query_pos,
                                   int qp_itype, const void* key_positions, int kp_itype, float* out,
                                   int batch, int64_t seq_len, int num_q_heads, int num_kv_heads,
                                   int d, int num_freqs, int coeff_bits, int pre_rope, void* workspace,
                                   size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(batch >= 0 && seq_len >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_tri_decode_step: bad sizes");
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_tri_decode_step: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(d > 0 && d % 2 == 0 && d <= 512, "akv_tri_decode_step: head_dim=%d must be even and <= 512", d);
  AKV_REQUIRE(num_freqs > 0 && num_freqs <= d / 2, "akv_tri_decode_step: num_freqs=%d out of range", num_freqs);
  AKV_REQUIRE(coeff_bits == 4 || coeff_bits == 8 || coeff_bits == 16,
              "akv_tri_decode_step: coeff_bits=%d, must be 4, 8 or 16", coeff_bits);
  AKV_REQUIRE(akv_valid_dtype(q_dtype), "akv_tri_decode_step: bad dtype");
  AKV_REQUIRE(!query_pos || akv_valid_itype(qp_itype), "akv_tri_decode_step: bad query_pos type");
  AKV_REQUIRE(!key_positions || akv_valid_itype(kp_itype), "akv_tri_decode_step: bad key_positions type");
  if (batch == 0) return AKV_OK;
  AKV_REQUIRE(query && out && theta, "akv_tri_decode_step: null pointer");
  if (seq_len == 0) {  // softmax over an empty axis: the reference's scatter-add leaves zeros
    tri_zero_kernel<<<64, 256, 0, stream>>>(out, (size_t)batch * num_q_heads * d);
    AKV_LAUNCH_CHECK("tri_zero_kernel");
    return AKV_OK;
  }
  AKV_REQUIRE(k_indices && k_coeffs && v_indices && v_coeffs, "akv_tri_decode_step: null cache pointer");
  AKV_REQUIRE(coeff_bits == 16 || (k_scales && v_scales), "akv_tri_decode_step: null scales");
  AKV_REQUIRE(coeff_bits != 16 || ((((uintptr_t)k_coeffs | (uintptr_t)v_coeffs) & 1) == 0),
              "akv_tri_decode_step: float16 coefficients must be 2-byte aligned");
  AKV_REQUIRE(workspace != nullptr, "akv_tri_decode_step: null workspace");
  if (workspace_bytes < akv_tri_decode_workspace_bytes(batch, num_q_heads, d))
    return akv_fail(AKV_ERR_WORKSPACE, "akv_tri_decode_step: workspace %zu < %zu bytes", workspace_bytes,
                    akv_tri_decode_workspace_bytes(batch, num_q_heads, d));
  tri_args a;
  a.query = query; a.q_dtype = q_dtype;
  a.k_idx = k_indices; a.k_cf = (const uint8_t*)k_coeffs; a.k_sc = (const __half*)k_scales;
  a.v_idx = v_indices; a.v_cf = (const uint8_t*)v_coeffs; a.v_sc = (const __half*)v_scales;
  a.theta = theta; a.qpos = query_pos; a.qp_itype = qp_itype; a.kpos = key_positions; a.kp_itype = kp_itype;
  a.B = batch; a.S = seq_len; a.QH = num_q_heads; a.KVH = num_kv_heads; a.D = d; a.F = num_freqs;
  a.cbits = coeff_bits; a.post_rope = pre_rope ? 0 : 1;
  a.nsplit = tri_pick_splits(batch, num_kv_heads, seq_len);
  a.block_tables = nullptr; a.bt_itype = AKV_I32; a.bt_stride = 0; a.context_lens = nullptr; a.cl_itype = AKV_I32;
  a.block_size = 0; a.num_blocks = 0; a.bs_shift = 0; a.bs_magic = 0; a.bs_mshift = 0; a.two_stages = 0;
  float* wsf = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  a.part_acc = wsf;
  a.part_ml = wsf + (size_t)batch * num_q_heads * a.nsplit * d;
  const int gqa = num_q_heads / num_kv_heads;
  // rows of 12 bytes can be read as dwords when the arrays are 4-byte aligned
  const bool wide = coeff_bits != 4;
  const bool f12 = !wide && num_freqs == 12 &&
                   ((((uintptr_t)k_indices | (uintptr_t)k_coeffs | (uintptr_t)v_indices | (uintptr_t)v_coeffs) & 3) == 0);
  const bool dense = d == 128;
  if (dense && f12 && num_kv_heads <= 8 && (uint64_t)seq_len * num_kv_heads * 12 < (1ull << 32)) {
    // one workgroup per (token range, batch element), a wavefront per kv head
    const int gq = gqa % 4 == 0 ? 4 : 1;
    const bool qh = q_dtype == AKV_F16;
    const bool two = tri_two_stages(num_kv_heads, gq, qh);
    const size_t lds = tri_roles_lds_bytes(num_kv_heads, gq, qh, two);
    if (lds <= 160 * 1024) {
      a.two_stages = two ? 1 : 0;
      int cus = akv_cached_cu_count();
      if (cus <= 0) cus = 256;
      const int passes = gqa / gq;
      int64_t n = (cus + batch * passes - 1) / (batch * passes);
      const int64_t by_len = (seq_len + 63) / 64;
      if (n > by_len) n = by_len;
      if (n > TRI_MAX_SPLITS) n = TRI_MAX_SPLITS;
      if (n < 1) n = 1;
      a.nsplit = (int)n;
      a.part_ml = wsf + (size_t)batch * num_q_heads * a.nsplit * d;
      dim3 hgrid(a.nsplit, batch, passes);
      if (key_positions) TRI_HEADS_LAUNCH(false, true, true); else TRI_HEADS_LAUNCH(false, false, true);
      AKV_LAUNCH_CHECK("tri_decode_heads_kernel");
      tri_reduce_kernel<<<batch * num_q_heads, 128, 0, stream>>>(a.part_acc, a.part_ml, a.nsplit, d, out);
      AKV_LAUNCH_CHECK("tri_reduce_kernel");
      return AKV_OK;
    }
  }
  dim3 grid(a.nsplit / TRI_WAVES, num_kv_heads, batch);
  akv_profile_mark_begin(stream);
#define TRI_LAUNCH(GQV)                                                                                   \
  do {                                                                                                    \
    const size_t per_wave = dense ? (size_t)(TRI_DENSE_WAVE_BYTES / 4) : (size_t)GQV * d;                 \
    const size_t lds = ((size_t)d / 2 + (size_t)GQV * d + (wide ? 256 : 16) + TRI_WAVES * per_wave) * sizeof(float); \
    if (dense) {   /* more than 64 KB of dynamic LDS has to be allowed once per kernel */               \
      static bool configured = false;                                                                     \
      if (!configured) {                                                                                  \
        const int most = (int)(lds + 240 * sizeof(float));                                                \
        AKV_HIP(hipFuncSetAttribute((const void*)tri_decode_kernel<GQV, true, true, false>,               \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, most));                   \
        AKV_HIP(hipFuncSetAttribute((const void*)tri_decode_kernel<GQV, false, true, false>,              \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, most));                   \
        AKV_HIP(hipFuncSetAttribute((const void*)tri_decode_kernel<GQV, false, true, true>,               \
                                    hipFuncAttributeMaxDynamicSharedMemorySize, most));                   \
        configured = true;                                                                                \
      }                                                                                                   \
    }                                                                                                     \
    if (dense && wide) tri_decode_kernel<GQV, false, true, true><<<grid, 256, lds, stream>>>(a);          \
    else if (wide) tri_decode_kernel<GQV, false, false, true><<<grid, 256, lds, stream>>>(a);             \
    else if (dense && f12) tri_decode_kernel<GQV, true, true, false><<<grid, 256, lds, stream>>>(a);      \
    else if (dense) tri_decode_kernel<GQV, false, true, false><<<grid, 256, lds, stream>>>(a);            \
    else if (f12) tri_decode_kernel<GQV, true, false, false><<<grid, 256, lds, stream>>>(a);              \
    else tri_decode_kernel<GQV, false, false, false><<<grid, 256, lds, stream>>>(a);                      \
  } while (0)
  if (gqa % 4 == 0) TRI_LAUNCH(4); else TRI_LAUNCH(1);
#undef TRI_LAUNCH
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("tri_decode_kernel");
  tri_reduce_kernel<<<batch * num_q_heads, 128, 0, stream>>>(a.part_acc, a.part_ml, a.nsplit, d, out);
  AKV_LAUNCH_CHECK("tri_reduce_kernel");
  return AKV_OK;
}

extern "C" int akv_tri_decode_paged(const void* query, int q_dtype, const uint8_t* k_indices,
                                    const uint8_t* k_coeffs, const void* k_scales,
                                    const uint8_t* v_indices, const uint8_t* v_coeffs,
                                    const void* v_scales, const float* theta, const void* query_pos,
                                    int qp_itype, const void* block_tables, int bt_itype,
                                    int64_t bt_stride, const void* context_lens, int cl_itype,
                                    float* out, int batch, int64_t num_blocks, int block_size,
                                    int64_t max_blocks_per_seq, int num_q_heads, int num_kv_heads,
                                    int d, int num_freqs, int pre_rope, void* workspace,
                                    size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(batch >= 0 && num_blocks > 0 && block_size > 0 && max_blocks_per_seq >= 0 && num_q_heads > 0 &&
              num_kv_heads > 0, "akv_tri_decode_paged: bad sizes");
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_tri_decode_paged: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(akv_valid_dtype(q_dtype), "akv_tri_decode_paged: bad dtype");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_tri_decode_paged: bad index type");
  AKV_REQUIRE(!query_pos || akv_valid_itype(qp_itype), "akv_tri_decode_paged: bad query_pos type");
  const bool aligned = ((((uintptr_t)k_indices | (uintptr_t)k_coeffs | (uintptr_t)v_indices | (uintptr_t)v_coeffs) & 3) == 0);
  const int gqa = num_q_heads / num_kv_heads;
  const int gq = gqa % 4 == 0 ? 4 : 1;
  const bool qh = q_dtype == AKV_F16;
  const bool two = tri_two_stages(num_kv_heads, gq, qh);
  const size_t lds = tri_roles_lds_bytes(num_kv_heads, gq, qh, two);
  if (d != 128 || num_freqs != 12 || num_kv_heads > 8 || !aligned || lds > 160 * 1024 ||
      max_blocks_per_seq * block_size >= ((int64_t)1 << 30) || block_size >= (1 << 30) ||
      (double)num_blocks * block_size * num_kv_heads >= 4294967296.0)
    return akv_fail(AKV_ERR_UNSUPPORTED,
                    "akv_tri_decode_paged: needs head_dim 128, 12 frequencies, at most 8 kv heads, 4-byte "
                    "aligned arrays, fewer than 2^30 tokens per sequence and fewer than 2^32 rows in the cache");
  // blocks of 1 .. 64 tokens (a power of two) in a cache whose arrays stay below 4 GB: rows by 32-bit offsets
  const bool bs_small = (block_size & (block_size - 1)) == 0 && block_size <= 64 && num_blocks < (1 << 24) &&
                        (double)num_blocks * block_size * num_kv_heads * 12.0 < 4294967296.0;
  if (!bs_small && block_size < 3)
    return akv_fail(AKV_ERR_UNSUPPORTED, "akv_tri_decode_paged: blocks of %d tokens in a cache of 4 GB arrays or more", block_size);
  if (batch == 0) return AKV_OK;
  AKV_REQUIRE(out != nullptr, "akv_tri_decode_paged: null pointer");
  if (max_blocks_per_seq == 0) {   // block tables without columns: every sequence is empty
    tri_zero_kernel<<<64, 256, 0, stream>>>(out, (size_t)batch * num_q_heads * d);
    AKV_LAUNCH_CHECK("tri_zero_kernel");
    return AKV_OK;
  }
  AKV_REQUIRE(query && theta && block_tables && context_lens, "akv_tri_decode_paged: null pointer");
  AKV_REQUIRE(k_indices && k_coeffs && k_scales && v_indices && v_coeffs && v_scales,
              "akv_tri_decode_paged: null cache pointer");
  AKV_REQUIRE(workspace != nullptr, "akv_tri_decode_paged: null workspace");
  if (workspace_bytes < akv_tri_decode_workspace_bytes(batch, num_q_heads, d))
    return akv_fail(AKV_ERR_WORKSPACE, "akv_tri_decode_paged: workspace %zu < %zu bytes", workspace_bytes,
                    akv_tri_decode_workspace_bytes(batch, num_q_heads, d));
  tri_args a;
  a.query = query; a.q_dtype = q_dtype;
  a.k_idx = k_indices; a.k_cf = k_coeffs; a.k_sc = (const __half*)k_scales;
  a.v_idx = v_indices; a.v_cf = v_coeffs; a.v_sc = (const __half*)v_scales;
  a.theta = theta; a.qpos = query_pos; a.qp_itype = qp_itype; a.kpos = nullptr; a.kp_itype = AKV_I32;
  a.B = batch; a.S = max_blocks_per_seq * block_size; a.QH = num_q_heads; a.KVH = num_kv_heads; a.D = d; a.F = num_freqs;
  a.cbits = 4; a.post_rope = pre_rope ? 0 : 1;
  a.block_tables = block_tables; a.bt_itype = bt_itype; a.bt_stride = bt_stride;
  a.context_lens = context_lens; a.cl_itype = cl_itype; a.block_size = block_size; a.num_blocks = num_blocks;
  a.two_stages = two ? 1 : 0;
  a.bs_shift = 0; a.bs_magic = 0; a.bs_mshift = 0;
  if (bs_small) {
    a.bs_shift = __builtin_ctz((unsigned)block_size);
  } else {
    // block_size >= 3 here: k = 30 + ceil(log2 block_size) >= 32 and magic = ceil(2^k / block_size) < 2^31
    const int k = 30 + (32 - __builtin_clz((unsigned)block_size - 1));
    a.bs_magic = (uint32_t)((((uint64_t)1 << k) + (uint64_t)block_size - 1) / (uint64_t)block_size);
    a.bs_mshift = k - 32;
  }
  int cus = akv_cached_cu_count();
  if (cus <= 0) cus = 256;
  const int passes = gqa / gq;
  int64_t n = (cus + batch * passes - 1) / (batch * passes);
  const int64_t by_len = (a.S + 63) / 64;
  if (n > by_len) n = by_len;
  if (n > TRI_MAX_SPLITS) n = TRI_MAX_SPLITS;
  if (n < 1) n = 1;
  a.nsplit = (int)n;
  float* wsf = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  a.part_acc = wsf;
  a.part_ml = wsf + (size_t)batch * num_q_heads * a.nsplit * d;
  dim3 hgrid(a.nsplit, batch, passes);
  if (bs_small) TRI_HEADS_LAUNCH(true, false, true);
  else TRI_HEADS_LAUNCH(true, false, false);
  AKV_LAUNCH_CHECK("tri_decode_heads_kernel");
  tri_reduce_kernel<<<batch * num_q_heads, 128, 0, stream>>>(a.part_acc, a.part_ml, a.nsplit, d, out);
  AKV_LAUNCH_CHECK("tri_reduce_kernel");
  return AKV_OK;
}

extern "C" int akv_tri_scores(const void* query, int q_dtype, const uint8_t* k_indices, const void* k_coeffs,
                              const void* k_scales, const float* theta, const void* query_pos, int qp_itype,
                              const void* key_positions, int kp_itype, float* out, int batch, int64_t seq_len,
                              int num_q_heads, int num_kv_heads, int d, int num_freqs, int coeff_bits, int pre_rope,
                              void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(batch >= 0 && seq_len >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_tri_scores: bad sizes");
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_tri_scores: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(d > 0 && d % 2 == 0 && d <= 512, "akv_tri_scores: head_dim=%d must be even and <= 512", d);
  AKV_REQUIRE(num_freqs > 0 && num_freqs <= d / 2, "akv_tri_scores: num_freqs=%d out of range", num_freqs);
  AKV_REQUIRE(coeff_bits == 4 || coeff_bits == 8 || coeff_bits == 16, "akv_tri_scores: coeff_bits=%d, must be 4, 8 or 16",
              coeff_bits);
  AKV_REQUIRE(akv_valid_dtype(q_dtype), "akv_tri_scores: bad dtype");
  AKV_REQUIRE(!query_pos || akv_valid_itype(qp_itype), "akv_tri_scores: bad query_pos type");
  AKV_REQUIRE(!key_positions || akv_valid_itype(kp_itype), "akv_tri_scores: bad key_positions type");
  if (batch == 0 || seq_len == 0) return AKV_OK;
  AKV_REQUIRE(query && out && theta && k_indices && k_coeffs, "akv_tri_scores: null pointer");
  AKV_REQUIRE(coeff_bits == 16 || k_scales, "akv_tri_scores: null scales");
  AKV_REQUIRE(coeff_bits != 16 || ((uintptr_t)k_coeffs & 1) == 0, "akv_tri_scores: float16 coefficients must be 2-byte aligned");
  AKV_REQUIRE((seq_len + 255) / 256 < ((int64_t)1 << 31) && num_kv_heads < 65536 && batch < 65536, "akv_tri_scores: grid too large");
  tri_args a = {};
  a.query = query; a.q_dtype = q_dtype;
  a.k_idx = k_indices; a.k_cf = (const uint8_t*)k_coeffs; a.k_sc = (const __half*)k_scales;
  a.theta = theta; a.qpos = query_pos; a.qp_itype = qp_itype; a.kpos = key_positions; a.kp_itype = kp_itype;
  a.B = batch; a.S = seq_len; a.QH = num_q_heads; a.KVH = num_kv_heads; a.D = d; a.F = num_freqs;
  a.cbits = coeff_bits; a.post_rope = pre_rope ? 0 : 1;
  const int gqa = num_q_heads / num_kv_heads;
  const int gq = gqa % 4 == 0 ? 4 : 1;
  const size_t lds = ((size_t)d / 2 + (size_t)gq * d + 256) * sizeof(float);
  dim3 grid((unsigned)((seq_len + 255) / 256), num_kv_heads, batch);
  if (gq == 4) tri_scores_kernel<4><<<grid, 256, lds, stream>>>(a, out);
  else tri_scores_kernel<1><<<grid, 256, lds, stream>>>(a, out);
  AKV_LAUNCH_CHECK("tri_scores_kernel");
  return AKV_OK;
}

// ----------------------------------------------------------------------------------
// SpectralKVEncoder.encode (aither_kvcache/triattention/encoder.py:73-149), coefficient widths 4 (a byte per
// pair, :118-133), 8 (two bytes per pair, :135-147) and 16 (the pair as two float16, scale 1, :107-115):
// one wavefront per vector, lane = RoPE pair.  A pair's rank is the number of pairs with larger
// energy (equal energies: lower index first; a NaN energy ranks above everything, as in
// torch.topk); pairs of rank < F are kept, their position in the ascending index order is the
// number of kept lanes below them.  Arithmetic follows the reference operation by operation
// (separately rounded squares and sum, true division by the scale, round half to even).
// ----------------------------------------------------------------------------------
// PAGED (encode-on-write): vector v is (token v / kvh, head v % kvh) of a [tokens][kv heads] tensor with
// element strides xs / xs_head, and its row goes to row slot x kvh + head of the block pool, slot =
// block x block_size + position from slot_mapping; tokens whose slot is negative or not below num_slots are skipped.
struct tri_enc_paged { int64_t xs_head; int kvh; const void* slots; int slot_itype; int64_t num_slots; };
template <int XDT, bool PAGED = false>
__global__ __launch_bounds__(256) void tri_encode_kernel(const void* __restrict__ x, int64_t n, int d, int64_t xs,
                                                         int F, int cbits, uint8_t* __restrict__ indices,
                                                         uint8_t* __restrict__ coeffs, __half* __restrict__ scales,
                                                         tri_enc_paged pg = {}) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // the same in every lane: the vector index and the search stay scalar
  const int P = d >> 1;
  const bool have = lane < P;
  const int64_t stride = (int64_t)gridDim.x * 4;
  // the lane's pair of a vector is requested one vector ahead
  auto fetch = [&](int64_t vv, float& p0, float& p1) {
    p0 = 0.f; p1 = 0.f;
    if (have && vv < n) {
      int64_t off = vv * xs;
      if constexpr (PAGED) {
        const int64_t tok = vv / pg.kvh;
        off = tok * xs + (vv - tok * pg.kvh) * pg.xs_head;
      }
      p0 = akv_elem<XDT>::load(x, off + 2 * lane);
      p1 = akv_elem<XDT>::load(x, off + 2 * lane + 1);
    }
  };
  float nx0, nx1;
  fetch((int64_t)blockIdx.x * 4 + wave, nx0, nx1);
  for (int64_t vsrc = (int64_t)blockIdx.x * 4 + wave; vsrc < n; vsrc += stride) {
    const float x0 = nx0, x1 = nx1;
    fetch(vsrc + stride, nx0, nx1);
    int64_t v = vsrc;               // row of the outputs
    if constexpr (PAGED) {
      const int64_t tok = vsrc / pg.kvh;
      const int64_t slot = akv_load_index(pg.slots, pg.slot_itype, tok);
      if (slot < 0 || slot >= pg.num_slots) continue;          // (wavefront-uniform)
      v = slot * pg.kvh + (vsrc - tok * pg.kvh);
    }
    const float e = akv_add_rn(akv_mul_rn(x0, x0), akv_mul_rn(x1, x1));
    // non-negative floats and NaNs order like their bit patterns; lanes beyond the last pair sort last
    const uint32_t key = have ? (__float_as_uint(e) & 0x7fffffffu) + 1u : 0u;
    // The F-th largest key by a bitwise search (largest T with at least F keys >= T: one compare and a
    // population count per bit), then everything above it plus, of the keys equal to it, the lowest
    // lanes -- the order torch.topk's result has once it is sorted by index with ties to the lower index.
    // (Once exactly F keys reach the threshold the remaining bits cannot change the set: the search stops there
    // -- looked at after every four bits --, after about half of its steps on keys without ties.  Written out
    // bit by bit, a step is one vector compare against a scalar and four scalar instructions.)
    uint32_t T = 0;
#pragma unroll
    for (int grp = 7; grp >= 0; --grp) {
#pragma unroll
      for (int b = 3; b >= 0; --b) {
        const uint32_t cand = T | (1u << (4 * grp + b));
        const int cnt = __builtin_popcountll(__builtin_amdgcn_ballot_w64(key >= cand));
        T = cnt >= F ? cand : T;
      }
      if (__builtin_popcountll(__builtin_amdgcn_ballot_w64(key >= T)) == F) break;
    }
    const bool above = key > T, equal = key == T;
    const int need = F - __popcll(__ballot(above));
    const uint64_t eqm = __ballot(equal);
    const int eq_pos = __builtin_amdgcn_mbcnt_hi((uint32_t)(eqm >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)eqm, 0u));
    const bool keep = have && (above || (equal && eq_pos < need));
    const uint64_t mask = __ballot(keep);
    const int pos = __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0u));
    float amax = keep ? fmaxf(fabsf(x0), fabsf(x1)) : 0.f;
    if (keep && (x0 != x0 || x1 != x1)) amax = __uint_as_float(0x7fc00000u);   // torch.amax propagates NaN
    // wave maximum that keeps a NaN: the values are non-negative or that one NaN pattern, which order like
    // their bit patterns with the NaN on top (lane rotations inside rows of sixteen, then the row swaps)
    uint32_t mb = __float_as_uint(amax);
    mb = max(mb, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mb, 0x128 /*row_ror:8*/, 0xf, 0xf, false));
    mb = max(mb, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mb, 0x124 /*row_ror:4*/, 0xf, 0xf, false));
    mb = max(mb, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mb, 0x122 /*row_ror:2*/, 0xf, 0xf, false));
    mb = max(mb, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)mb, 0x121 /*row_ror:1*/, 0xf, 0xf, false));
    {
      auto r32 = __builtin_amdgcn_permlane32_swap(mb, mb, false, false);
      mb = max(r32[0], r32[1]);
      auto r16 = __builtin_amdgcn_permlane16_swap(mb, mb, false, false);
      mb = max(r16[0], r16[1]);
    }
    const float m = __uint_as_float(mb);
    const float scale = (m != m) ? m : fmaxf(m, 1e-8f);
    if (keep && cbits == 16) {
      indices[v * F + pos] = (uint8_t)lane;
      ((__half*)coeffs)[(v * F + pos) * 2] = __float2half_rn(x0);
      ((__half*)coeffs)[(v * F + pos) * 2 + 1] = __float2half_rn(x1);
    } else if (keep) {
      const float half_code = cbits == 8 ? 127.5f : 7.5f, top = cbits == 8 ? 255.f : 15.f;
      const float c0 = rintf(akv_mul_rn(akv_add_rn(__fdiv_rn(x0, scale), 1.0f), half_code));
      const float c1 = rintf(akv_mul_rn(akv_add_rn(__fdiv_rn(x1, scale), 1.0f), half_code));
      // clamp(0, top) then the cast to uint8; a NaN becomes 0 as in torch's float -> uint8 conversion on the CPU
      const uint32_t q0 = c0 != c0 ? 0u : (uint32_t)fminf(fmaxf(c0, 0.f), top);
      const uint32_t q1 = c1 != c1 ? 0u : (uint32_t)fminf(fmaxf(c1, 0.f), top);
      indices[v * F + pos] = (uint8_t)lane;
      if (cbits == 8) {
        coeffs[(v * F + pos) * 2] = (uint8_t)q0;
        coeffs[(v * F + pos) * 2 + 1] = (uint8_t)q1;
      } else {
        coeffs[v * F + pos] = (uint8_t)((q0 << 4) | q1);
      }
    }
    if (lane == 0) scales[v] = cbits == 16 ? __float2half_rn(1.0f) : __float2half_rn(scale);
  }
}

extern "C" int akv_tri_encode(const void* x, int x_dtype, int64_t n, int d, int64_t x_stride, int num_freqs,
                              int coeff_bits, uint8_t* indices, void* coeffs, void* scales, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(n >= 0, "akv_tri_encode: n=%lld", (long long)n);
  AKV_REQUIRE(akv_valid_dtype(x_dtype), "akv_tri_encode: bad dtype");
  AKV_REQUIRE(d > 0 && d % 2 == 0, "akv_tri_encode: head_dim=%d must be even", d);
  AKV_REQUIRE(num_freqs > 0 && num_freqs <= d / 2, "akv_tri_encode: num_freqs=%d out of range", num_freqs);
  AKV_REQUIRE(coeff_bits == 4 || coeff_bits == 8 || coeff_bits == 16, "akv_tri_encode: coeff_bits=%d, must be 4, 8 or 16",
              coeff_bits);
  if (d > 128) return akv_fail(AKV_ERR_UNSUPPORTED, "akv_tri_encode: head_dim=%d above 128 (one lane per pair)", d);
  if (n == 0) return AKV_OK;
  AKV_REQUIRE(x && indices && coeffs && scales, "akv_tri_encode: null pointer");
  AKV_REQUIRE(x_stride >= d, "akv_tri_encode: stride smaller than row");
  AKV_REQUIRE(coeff_bits != 16 || ((uintptr_t)coeffs & 1) == 0, "akv_tri_encode: float16 coefficients must be 2-byte aligned");
  const int64_t want = (n + 3) / 4;
  const int cap = akv_cached_cu_count() * 32;
  const int grid = (int)(want < cap ? want : cap);
  switch (x_dtype) {
    case AKV_F16: tri_encode_kernel<AKV_F16><<<grid, 256, 0, stream>>>(x, n, d, x_stride, num_freqs, coeff_bits, indices, (uint8_t*)coeffs, (__half*)scales); break;
    case AKV_BF16: tri_encode_kernel<AKV_BF16><<<grid, 256, 0, stream>>>(x, n, d, x_stride, num_freqs, coeff_bits, indices, (uint8_t*)coeffs, (__half*)scales); break;
    default: tri_encode_kernel<AKV_F32><<<grid, 256, 0, stream>>>(x, n, d, x_stride, num_freqs, coeff_bits, indices, (uint8_t*)coeffs, (__half*)scales); break;
  }
  AKV_LAUNCH_CHECK("tri_encode_kernel");
  return AKV_OK;
}

// SpectralKVEncoder.encode of a step's K or V vectors written straight into the block pool of a paged spectral
// cache (SpectralKVCache.store_token, aither_kvcache/triattention/cache.py:106-140, for every token of the step at
// once): int4 coefficients, the only width that cache stores.
extern "C" int akv_tri_encode_paged(const void* x, int x_dtype, int64_t num_tokens, int num_kv_heads, int d,
                                    int64_t xs_token, int64_t xs_head, int num_freqs, const void* slot_mapping,
                                    int slot_itype, int64_t num_slots, uint8_t* indices, uint8_t* coeffs,
                                    void* scales, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(num_tokens >= 0 && num_kv_heads > 0 && num_slots >= 0, "akv_tri_encode_paged: bad sizes");
  AKV_REQUIRE(akv_valid_dtype(x_dtype) && akv_valid_itype(slot_itype), "akv_tri_encode_paged: bad dtype");
  AKV_REQUIRE(d > 0 && d % 2 == 0, "akv_tri_encode_paged: head_dim=%d must be even", d);
  AKV_REQUIRE(num_freqs > 0 && num_freqs <= d / 2, "akv_tri_encode_paged: num_freqs=%d out of range", num_freqs);
  if (d > 128) return akv_fail(AKV_ERR_UNSUPPORTED, "akv_tri_encode_paged: head_dim=%d above 128 (one lane per pair)", d);
  if (num_tokens == 0 || num_slots == 0) return AKV_OK;
  AKV_REQUIRE(x && slot_mapping && indices && coeffs && scales, "akv_tri_encode_paged: null pointer");
  AKV_REQUIRE(xs_head >= d && xs_token >= d, "akv_tri_encode_paged: stride smaller than row");
  const int64_t n = num_tokens * num_kv_heads;
  const int64_t want = (n + 3) / 4;
  const int cap = akv_cached_cu_count() * 32;
  const int grid = (int)(want < cap ? want : cap);
  tri_enc_paged pg;
  pg.xs_head = xs_head; pg.kvh = num_kv_heads; pg.slots = slot_mapping; pg.slot_itype = slot_itype; pg.num_slots = num_slots;
  switch (x_dtype) {
    case AKV_F16: tri_encode_kernel<AKV_F16, true><<<grid, 256, 0, stream>>>(x, n, d, xs_token, num_freqs, 4, indices, coeffs, (__half*)scales, pg); break;
    case AKV_BF16: tri_encode_kernel<AKV_BF16, true><<<grid, 256, 0, stream>>>(x, n, d, xs_token, num_freqs, 4, indices, coeffs, (__half*)scales, pg); break;
    default: tri_encode_kernel<AKV_F32, true><<<grid, 256, 0, stream>>>(x, n, d, xs_token, num_freqs, 4, indices, coeffs, (__half*)scales, pg); break;
  }
  AKV_LAUNCH_CHECK("tri_encode_kernel");
  return AKV_OK;
}
