// TriAttention decode_step (aither_kvcache/triattention/attention.py:186-280 with
// TrigSeriesScorer.score, scorer.py:115-208), int4 coefficients.
//
// Per (batch, kv head) the S cached tokens are cut into NSPLIT contiguous ranges, one
// wavefront each.  Lanes <-> tokens: a lane unpacks its token's F retained pairs, forms
//   c_f = q_e k0 + q_o k1,  s_f = q_o k0 - q_e k1   at the pair's index,
//   score = (1/sqrt(d)) sum_f (c_f cos(delta theta_f) + s_f sin(delta theta_f)),
// with delta = float(key_pos) - float(query_pos) and the phase formed by ONE float32 multiply
// as the reference does (phases reach ~3e4 rad, so the argument must match to the last bit
// before sin/cos).  The phases are shared by the GQ query heads of the kv head.  A running
// softmax is kept per wavefront; the weighted value coefficients are scatter-added into the
// wavefront's private LDS bins (D floats per query head).  A second kernel merges the NSPLIT
// partials with the log-sum-exp rule and writes float32.
#include "akv_common.h"

#define TRI_MAX_SPLITS 128
#define TRI_WAVES 4

struct tri_args {
  const void* query; int q_dtype;
  const uint8_t* k_idx; const uint8_t* k_cf; const __half* k_sc;
  const uint8_t* v_idx; const uint8_t* v_cf; const __half* v_sc;
  const float* theta;
  const void* qpos; int qp_itype;
  const void* kpos; int kp_itype;
  int B; int64_t S; int QH, KVH, D, F;
  int nsplit;
  float* part_acc;  // [B][QH][nsplit][D]
  float* part_ml;   // [B][QH][nsplit][2]
};

__device__ __forceinline__ float tri_dequant(uint32_t code, float scale) {
  // (code / 7.5 - 1) * scale, scorer.py:99-104
  return __fmul_rn(__fsub_rn(__fdiv_rn((float)code, 7.5f), 1.0f), scale);
}

template <int GQ>
__global__ __launch_bounds__(256) void tri_decode_kernel(tri_args a) {
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* theta = (float*)lds_raw;                         // [D/2]
  float* q_lds = theta + a.D / 2;                         // [GQ][D]   (per workgroup pass)
  float* acc_base = q_lds + GQ * a.D;                     // [TRI_WAVES][GQ][D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* acc = acc_base + (size_t)wave * GQ * a.D;
  const int D = a.D, F = a.F;
  const int gqa = a.QH / a.KVH;
  const int b = blockIdx.z, h = blockIdx.y;
  const int split = blockIdx.x * TRI_WAVES + wave;
  const float inv_sqrt_d = 1.0f / sqrtf((float)D);

  for (int i = threadIdx.x; i < D / 2; i += 256) theta[i] = a.theta[i];

  const int64_t per = (a.S + a.nsplit - 1) / a.nsplit;
  const int64_t s0 = min(a.S, (int64_t)split * per);
  const int64_t s1 = min(a.S, s0 + per);
  const float qp = a.qpos ? (float)akv_load_index(a.qpos, a.qp_itype, b) : (float)a.S;

  for (int qg = 0; qg < gqa; qg += GQ) {
    __syncthreads();
    for (int i = threadIdx.x; i < GQ * D; i += 256) {
      const int q = i / D, d = i % D;
      const int64_t off = ((int64_t)b * a.QH + (h * gqa + qg + q)) * D + d;
      float v;
      if (a.q_dtype == AKV_F16) v = akv_elem<AKV_F16>::load(a.query, off);
      else if (a.q_dtype == AKV_BF16) v = akv_elem<AKV_BF16>::load(a.query, off);
      else v = akv_elem<AKV_F32>::load(a.query, off);
      q_lds[i] = v;
    }
    for (int i = lane; i < GQ * D; i += 64) acc[i] = 0.f;
    __syncthreads();

    float m[GQ], l[GQ];
#pragma unroll
    for (int q = 0; q < GQ; ++q) { m[q] = -INFINITY; l[q] = 0.f; }

    for (int64_t c0 = s0; c0 < s1; c0 += 64) {
      const int64_t t = c0 + lane;
      const bool valid = t < s1;
      const int64_t tc = valid ? t : s1 - 1;
      const int64_t row = ((int64_t)b * a.S + tc) * a.KVH + h;
      const float kp = a.kpos ? (float)akv_load_index(a.kpos, a.kp_itype, (int64_t)b * a.S + tc) : (float)tc;
      const float delta = __fsub_rn(kp, qp);
      const float ksc = __half2float(a.k_sc[row]);
      float sc[GQ];
#pragma unroll
      for (int q = 0; q < GQ; ++q) sc[q] = 0.f;
      for (int f = 0; f < F; ++f) {
        const uint32_t idx = a.k_idx[row * F + f];
        const uint32_t cf = a.k_cf[row * F + f];
        const float k0 = tri_dequant(cf >> 4, ksc), k1 = tri_dequant(cf & 15u, ksc);
        const float ph = __fmul_rn(delta, theta[idx]);
        float sn, cs;
        sincosf(ph, &sn, &cs);
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const float qe = q_lds[q * D + 2 * idx], qo = q_lds[q * D + 2 * idx + 1];
          const float c = qe * k0 + qo * k1;
          const float s = qo * k0 - qe * k1;
          sc[q] += c * cs + s * sn;
        }
      }
      float p[GQ];
      bool rescale = false;
      float alpha[GQ];
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const float sv = valid ? sc[q] * inv_sqrt_d : -INFINITY;
        const float mn = fmaxf(m[q], akv_wave_max(sv));
        alpha[q] = __expf(m[q] - mn);
        rescale |= (mn != m[q]);
        p[q] = valid ? __expf(sv - mn) : 0.f;
        l[q] = l[q] * alpha[q] + p[q];
        m[q] = mn;
      }
      if (rescale) {  // wavefront-uniform: m is the same in every lane
#pragma unroll
        for (int q = 0; q < GQ; ++q)
          for (int i = lane; i < D; i += 64) acc[q * D + i] *= alpha[q];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
      if (valid) {
        const float vsc = __half2float(a.v_sc[row]);
        for (int f = 0; f < F; ++f) {
          const uint32_t idx = a.v_idx[row * F + f];
          const uint32_t cf = a.v_cf[row * F + f];
          const float v0 = tri_dequant(cf >> 4, vsc), v1 = tri_dequant(cf & 15u, vsc);
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
    if (split < a.nsplit) {
#pragma unroll
      for (int q = 0; q < GQ; ++q) {
        const size_t slot = ((size_t)b * a.QH + (h * gqa + qg + q)) * a.nsplit + split;
        const float lsum = akv_wave_sum(l[q]);
        for (int i = lane; i < D; i += 64) a.part_acc[slot * D + i] = acc[q * D + i];
        if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
      }
    }
  }
}

__global__ __launch_bounds__(64) void tri_reduce_kernel(const float* __restrict__ part_acc,
                                                        const float* __restrict__ part_ml,
                                                        int nsplit, int D, float* __restrict__ out) {
  const size_t pair = blockIdx.x;  // b * QH + qh
  const int lane = threadIdx.x;
  float m = -INFINITY;
  for (int s = 0; s < nsplit; ++s) m = fmaxf(m, part_ml[(pair * nsplit + s) * 2]);
  float l = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float ms = part_ml[(pair * nsplit + s) * 2];
    if (ms > -INFINITY) l += __expf(ms - m) * part_ml[(pair * nsplit + s) * 2 + 1];
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
  for (int i = lane; i < D; i += 64) {
    float acc = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float ms = part_ml[(pair * nsplit + s) * 2];
      if (ms > -INFINITY) acc += __expf(ms - m) * part_acc[(pair * nsplit + s) * D + i];
    }
    out[pair * D + i] = acc * inv;
  }
}

__global__ void tri_zero_kernel(float* out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) out[i] = 0.f;
}

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
                                   const uint8_t* k_coeffs, const void* k_scales,
                                   const uint8_t* v_indices, const uint8_t* v_coeffs,
                                   const void* v_scales, const float* theta, const void* query_pos,
                                   int qp_itype, const void* key_positions, int kp_itype, float* out,
                                   int batch, int64_t seq_len, int num_q_heads, int num_kv_heads,
                                   int d, int num_freqs, void* workspace, size_t workspace_bytes,
                                   void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(batch >= 0 && seq_len >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_tri_decode_step: bad sizes");
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_tri_decode_step: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(d > 0 && d % 2 == 0 && d <= 512, "akv_tri_decode_step: head_dim=%d must be even and <= 512", d);
  AKV_REQUIRE(num_freqs > 0 && num_freqs <= d / 2, "akv_tri_decode_step: num_freqs=%d out of range", num_freqs);
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
  AKV_REQUIRE(k_indices && k_coeffs && k_scales && v_indices && v_coeffs && v_scales,
              "akv_tri_decode_step: null cache pointer");
  AKV_REQUIRE(workspace != nullptr, "akv_tri_decode_step: null workspace");
  if (workspace_bytes < akv_tri_decode_workspace_bytes(batch, num_q_heads, d))
    return akv_fail(AKV_ERR_WORKSPACE, "akv_tri_decode_step: workspace %zu < %zu bytes", workspace_bytes,
                    akv_tri_decode_workspace_bytes(batch, num_q_heads, d));
  tri_args a;
  a.query = query; a.q_dtype = q_dtype;
  a.k_idx = k_indices; a.k_cf = k_coeffs; a.k_sc = (const __half*)k_scales;
  a.v_idx = v_indices; a.v_cf = v_coeffs; a.v_sc = (const __half*)v_scales;
  a.theta = theta; a.qpos = query_pos; a.qp_itype = qp_itype; a.kpos = key_positions; a.kp_itype = kp_itype;
  a.B = batch; a.S = seq_len; a.QH = num_q_heads; a.KVH = num_kv_heads; a.D = d; a.F = num_freqs;
  a.nsplit = tri_pick_splits(batch, num_kv_heads, seq_len);
  float* wsf = (float*)(((uintptr_t)workspace + 255) & ~(uintptr_t)255);
  a.part_acc = wsf;
  a.part_ml = wsf + (size_t)batch * num_q_heads * a.nsplit * d;
  const int gqa = num_q_heads / num_kv_heads;
  dim3 grid(a.nsplit / TRI_WAVES, num_kv_heads, batch);
  akv_profile_mark_begin(stream);
  if (gqa % 4 == 0) {
    const size_t lds = ((size_t)d / 2 + 4 * d + TRI_WAVES * 4 * d) * sizeof(float);
    tri_decode_kernel<4><<<grid, 256, lds, stream>>>(a);
  } else {
    const size_t lds = ((size_t)d / 2 + 1 * d + TRI_WAVES * 1 * d) * sizeof(float);
    tri_decode_kernel<1><<<grid, 256, lds, stream>>>(a);
  }
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("tri_decode_kernel");
  tri_reduce_kernel<<<batch * num_q_heads, 64, 0, stream>>>(a.part_acc, a.part_ml, a.nsplit, d, out);
  AKV_LAUNCH_CHECK("tri_reduce_kernel");
  return AKV_OK;
}
