// Paged decode attention over a uniform TurboQuant cache (2/3/4-bit):
//   prologue  : q' = Pi q for every (sequence, query head) + per-sequence block prefix
//   main      : stream-K walk over (sequence, block) pairs, all kv heads per workgroup
//   reduce    : log-sum-exp merge of the partials, /l, out = Pi^T a, cast
// This file holds the prologue, the reduce and the general main kernel (any of the three
// bit widths, head_dim 64/128/256).  The MFMA main kernel for 4-bit / head_dim 128 is in
// akv_attn_mfma.hip and plugs into the same prologue / reduce.
#include "akv_attn_common.h"


// ----------------------------------------------------------------------------------
// prologue
// ----------------------------------------------------------------------------------
template <int QDT>
__global__ __launch_bounds__(256) void akv_attn_prologue_kernel(
    const void* __restrict__ query, int64_t qs_seq, int64_t qs_head, const float* __restrict__ PiT,
    int S, int QH, int D, const void* context_lens, int cl_itype, int block_size,
    int64_t max_blocks_per_seq, int32_t* prefix, float* __restrict__ qrot, uint32_t* __restrict__ status) {
  __shared__ float q_lds[512];
  __shared__ int32_t scratch[257];
  const int b = blockIdx.x;
  if (b == S * QH) {
    if (threadIdx.x == 0) status[0] = 0u;
    akv_block_prefix_scan(context_lens, cl_itype, S, block_size, max_blocks_per_seq, prefix, scratch);
    return;
  }
  const int s = b / QH, h = b % QH;
  const int tid = threadIdx.x;
  for (int t = tid; t < D; t += 256) q_lds[t] = akv_elem<QDT>::load(query, s * qs_seq + h * qs_head + t);
  __syncthreads();
  for (int t = tid; t < D; t += 256) {
    float acc = 0.f;
    for (int j = 0; j < D; ++j) acc = fmaf(PiT[(size_t)j * D + t], q_lds[j], acc);
    qrot[((size_t)s * QH + h) * D + t] = acc;
  }
}

// ----------------------------------------------------------------------------------
// reduce: a workgroup takes (sequence, group of 4 query heads) items, blockIdx.x, + gridDim.x, ...
// Wavefront w merges the partials of head 4*group + w; then all 256 threads apply the inverse
// rotation, one load of Pi[k][j] serving two heads.  At head_dim 128 a thread keeps its column of
// Pi in registers across its items: with one workgroup per item a batch of 256 sequences x 32 heads
// read the 64 KB matrix 4096 times (43 us for the kernel; 2048 items on 512 workgroups: see the host side).
// ----------------------------------------------------------------------------------
template <int D, int ODT>
__global__ __launch_bounds__(256, 3) void akv_attn_reduce_kernel(
    const int32_t* __restrict__ prefix, const float* __restrict__ part_acc,
    const float* __restrict__ part_ml, const float* __restrict__ Pi, const uint4* __restrict__ bop, int S, int QH, int G,
    void* __restrict__ out, int64_t os_seq, int64_t os_head, const uint32_t* __restrict__ status,
    const int32_t* __restrict__ seqw) {
  constexpr int DPL = D / 64;
  __shared__ __align__(16) float a_lds[4][D + 8];    // (rows 8 banks apart: the four heads are read together)
  const int groups = (QH + 3) / 4;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // head_dim 128: the inverse rotation runs on the matrix cores.  Wavefront w owns N-tiles 2w and 2w + 1 of the
  // matrix operand (output coordinates 8 col + N-tile: lane col ends up with the neighbouring coordinates
  // 8 col + 2w and + 1); its 16 operand registers per term are requested before anything else and stay for
  // all items of the workgroup.  (On the vector unit, with a column of the matrix per thread, the rotation was
  // 22 of the kernel's 39 us for 256 sequences x 32 heads.)
  akv_half8 bh[2][4], bl[2][4];
  if constexpr (D == 128) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int idx = ((2 * wave + t) * 4 + ks) * 64 + lane;
        bh[t][ks] = akv_as_half8(bop[idx]);
        bl[t][ks] = akv_as_half8(bop[2048 + idx]);
      }
  }
  // a main kernel whose bounded wait gave up has produced garbage: say so in every output
  const float poison = status[0] != 0u ? __uint_as_float(0x7fc00000u) : 0.f;
  for (int item = blockIdx.x; item < S * groups; item += gridDim.x) {
  const int s = item / groups, hg = item % groups;
  const int h = hg * 4 + wave;
  // workgroups of the main kernel whose ranges meet the sequence: from the record of the matrix-core
  // kernel's prologue (seqw), else from the equal cut of the block axis
  int b0 = 0, b1 = 0, w_lo, w_hi;
  if (seqw != nullptr) {
    w_lo = seqw[2 * s];
    w_hi = seqw[2 * s + 1];
  } else {
    b0 = prefix[s];
    b1 = prefix[s + 1];
    const int per = (prefix[S] + G - 1) / G;
    w_lo = per > 0 ? b0 / per : 0;
    w_hi = b1 > b0 ? (b1 - 1) / per : w_lo - 1;
  }
  if (w_hi < w_lo) {        // an empty sequence (the same for the whole workgroup)
    if (h < QH) {
#pragma unroll
      for (int i = 0; i < DPL; ++i) akv_elem<ODT>::store(out, s * os_seq + h * os_head + lane * DPL + i, poison);
    }
    continue;
  }
  if (h < QH) {
    // the first RED_PF partial accumulators are requested before anything is known about their
    // weights, so that their round trip overlaps the one of the (max, sum) pairs
    // (only slots that exist are read: a batch of many short sequences has one or two per head)
    constexpr int RED_PF = D == 128 ? 32 : 16;
    float pre[RED_PF][DPL];
#pragma unroll
    for (int u = 0; u < RED_PF; ++u) {
      if (w_lo + u <= w_hi) {
        const size_t slot = (size_t)(w_lo + u + s) * QH + h;
#pragma unroll
        for (int i = 0; i < DPL; ++i) pre[u][i] = part_acc[slot * D + lane * DPL + i];
      } else {
#pragma unroll
        for (int i = 0; i < DPL; ++i) pre[u][i] = 0.f;
      }
    }
    // lanes over slots: global max and sum; with at most 64 slots (the usual case) lane u keeps the
    // weight of slot w_lo + u and the second pass takes it from there
    const bool few = w_hi - w_lo < 64;
    float M = -INFINITY, ms0 = -INFINITY, ls0 = 0.f;
    for (int w = w_lo + lane; w <= w_hi; w += 64) {
      const size_t slot = (size_t)(w + s) * QH + h;
      const float2 ml = *(const float2*)(part_ml + slot * 2);
      if (w < w_lo + 64) { ms0 = ml.x; ls0 = ml.y; }
      M = fmaxf(M, ml.x);
    }
    M = akv_wave_max(M);
    const float wgt0 = ms0 > -INFINITY ? __expf(ms0 - M) : 0.f;
    float l = wgt0 * ls0;
    for (int w = w_lo + 64 + lane; w <= w_hi; w += 64) {
      const size_t slot = (size_t)(w + s) * QH + h;
      const float ms = part_ml[slot * 2];
      if (ms > -INFINITY) l += __expf(ms - M) * part_ml[slot * 2 + 1];
    }
    l = akv_wave_sum(l);
    float acc[DPL];
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[i] = 0.f;
#pragma unroll
    for (int u = 0; u < RED_PF; ++u) {
      const float wu = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wgt0), u));
      const float wgt = (w_lo + u <= w_hi) ? wu : 0.f;
#pragma unroll
      for (int i = 0; i < DPL; ++i) acc[i] = fmaf(wgt, pre[u][i], acc[i]);
    }
    if (few) {
      // batches of eight independent loads (a batch past the end repeats the last slot with weight 0)
      for (int w0 = w_lo + RED_PF; w0 <= w_hi; w0 += 8) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const int w = min(w0 + u, w_hi);
          const size_t slot = (size_t)(w + s) * QH + h;
          const float wl = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(wgt0), w - w_lo));
          const float wgt = (w0 + u <= w_hi) ? wl : 0.f;
#pragma unroll
          for (int i = 0; i < DPL; ++i) acc[i] = fmaf(wgt, part_acc[slot * D + lane * DPL + i], acc[i]);
        }
      }
    } else {
#pragma unroll 8
      for (int w = w_lo + RED_PF; w <= w_hi; ++w) {
        const size_t slot = (size_t)(w + s) * QH + h;
        const float ms = part_ml[slot * 2];
        const float wgt = ms > -INFINITY ? __expf(ms - M) : 0.f;
#pragma unroll
        for (int i = 0; i < DPL; ++i) acc[i] = fmaf(wgt, part_acc[slot * D + lane * DPL + i], acc[i]);
      }
    }
    const float inv = l > 0.f ? 1.f / l : 1.f;
#pragma unroll
    for (int i = 0; i < DPL; ++i) a_lds[wave][lane * DPL + i] = acc[i] * inv;
  } else {
#pragma unroll
    for (int i = 0; i < DPL; ++i) a_lds[wave][lane * DPL + i] = 0.f;
  }
  __syncthreads();
  if constexpr (D == 128) {
    // A operand: row r = head r % 4 of the item (rows 4..15 repeat them and are not used), contracted coordinates
    // 32 kg + 8 ks + e of the merged vector; result: lane (col, 0) holds heads 0..3 for output coordinates
    // 8 col + 2 wave and + 1
    const int r = lane & 15, kg = lane >> 4;
    float v[4][8];
    float m = 0.f;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const float4 x0 = *(const float4*)&a_lds[r & 3][32 * kg + 8 * ks];
      const float4 x1 = *(const float4*)&a_lds[r & 3][32 * kg + 8 * ks + 4];
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
    const float usc = akv_row_unscale(ex) * (1.f / 64.f);     // lane i < 4: the factor of head i
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float ui = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(usc), i));
      const int hq = hg * 4 + i;
      if (kg == 0 && hq < QH) {
        akv_elem<ODT>::store(out, s * os_seq + hq * os_head + 8 * r + 2 * wave, acc[0][i] * ui + poison);
        akv_elem<ODT>::store(out, s * os_seq + hq * os_head + 8 * r + 2 * wave + 1, acc[1][i] * ui + poison);
      }
    }
  } else {
  // inverse rotation: thread t owns coordinates (t % 128) * JP .. of heads 2 * (t / 128) and + 1
  constexpr int JT = 128;                 // threads along the coordinate axis
  constexpr int JP = D / JT > 0 ? D / JT : 1;   // coordinates per thread (D=256 -> 2)
  const int jt = threadIdx.x % JT, pr = threadIdx.x / JT;
  if (jt * JP < D) {
    float o[2][JP];
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int i = 0; i < JP; ++i) o[q][i] = 0.f;
#pragma unroll 64
    for (int k = 0; k < D; ++k) {
      const float a0v = a_lds[2 * pr][k], a1v = a_lds[2 * pr + 1][k];
#pragma unroll
      for (int i = 0; i < JP; ++i) {
        const float pv = Pi[(size_t)k * D + jt * JP + i];
        o[0][i] = fmaf(a0v, pv, o[0][i]);
        o[1][i] = fmaf(a1v, pv, o[1][i]);
      }
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int hq = hg * 4 + 2 * pr + q;
      if (hq < QH) {
#pragma unroll
        for (int i = 0; i < JP; ++i)
          akv_elem<ODT>::store(out, s * os_seq + hq * os_head + jt * JP + i, o[q][i] + poison);
      }
    }
  }
  }
  __syncthreads();       // the merged vectors are read until here; the next item overwrites them
  }
}

// ----------------------------------------------------------------------------------
// general main kernel: 8 wavefronts, wavefront <-> kv head.  Per 64-token chunk a wavefront
// first scores with lanes <-> tokens (packed K row in registers, q' broadcast from LDS),
// updates the running softmax, then accumulates V with lanes <-> coordinates (V rows and
// weights staged in the wavefront's own LDS slice).  The query heads of a kv head are taken
// GQ at a time (GQ = 4 when the GQA ratio is a multiple of 4, else 1).
// ----------------------------------------------------------------------------------
#define AKV_ATTN_WAVES 8      // wavefronts of a workgroup (4 at head_dim 512, where a wavefront's staging area is four times as large)
template <int D> constexpr int akv_attn_gen_waves() { return D >= 512 ? 4 : AKV_ATTN_WAVES; }

template <int D, int BITS, int GQ>
struct akv_attn_gen_cfg {
  static constexpr int ROWDW = D * BITS / 32;
  static constexpr int VROW = ROWDW + 1;  // padded row stride in dwords
  static constexpr size_t wave_floats = 64 * GQ + 64 * VROW;
  static size_t lds_bytes(int QH) { return ((size_t)QH * D + akv_attn_gen_waves<D>() * wave_floats + 16) * 4; }
};

template <int D, int BITS, int GQ>
__global__ __launch_bounds__(512) void akv_attn_general_kernel(akv_attn_args a) {
  typedef akv_attn_gen_cfg<D, BITS, GQ> cfg;
  constexpr int DPL = D / 64;
  constexpr int ROWDW = cfg::ROWDW;
  constexpr int VROW = cfg::VROW;
  extern __shared__ __align__(16) unsigned char lds_raw[];
  float* q_lds = (float*)lds_raw;                          // [QH][D]
  float* wave_base = q_lds + (size_t)a.QH * D;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float* p_lds = wave_base + wave * cfg::wave_floats;      // [64][GQ]
  uint32_t* v_lds = (uint32_t*)(p_lds + 64 * GQ);          // [64][VROW]
  float* cen = wave_base + akv_attn_gen_waves<D>() * cfg::wave_floats;

  if (threadIdx.x < (1 << BITS)) cen[threadIdx.x] = a.centroids[threadIdx.x];

  const int G = gridDim.x;
  const int total = a.prefix[a.S];
  const int per = (total + G - 1) / G;
  const int g0 = blockIdx.x * per;
  const int g1 = min(total, g0 + per);
  const int gqa = a.QH / a.KVH;
  const int bs = a.block_size;

  int g = g0;
  while (g < g1) {
    const int s = akv_find_seq(a.prefix, a.S, g);
    const int sb0 = a.prefix[s], sb1 = a.prefix[s + 1];
    const int blk_lo = g - sb0;
    const int blk_hi = min(g1, sb1) - sb0;
    const int64_t ctx = akv_seq_tokens(a.context_lens, a.cl_itype, s, bs, a.max_blocks_per_seq);
    const int t0 = blk_lo * bs;
    const int t1 = (int)min((int64_t)blk_hi * bs, ctx);
    g = sb0 + blk_hi;

    __syncthreads();  // previous segment done with q_lds
    for (int i = threadIdx.x; i < a.QH * D; i += blockDim.x)
      q_lds[i] = a.qrot[(size_t)s * a.QH * D + i];
    __syncthreads();

    for (int h = wave; h < a.KVH; h += akv_attn_gen_waves<D>()) {
      for (int qg = 0; qg < gqa; qg += GQ) {
        float m[GQ], l[GQ], acc[GQ][DPL];
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          m[q] = -INFINITY; l[q] = 0.f;
#pragma unroll
          for (int i = 0; i < DPL; ++i) acc[q][i] = 0.f;
        }
        const float* qh = q_lds + (size_t)(h * gqa + qg) * D;

        for (int c0 = t0; c0 < t1; c0 += 64) {
          const int t = c0 + lane;
          const bool valid = t < t1;
          const int tc = valid ? t : t1 - 1;
          const int64_t phys = akv_clamp_block(akv_load_index(a.block_tables, a.bt_itype, s * a.bt_stride + tc / bs), a.num_blocks);
          const int pos = tc % bs;
          // ---- scores: lanes <-> tokens; 32 coordinates (= BITS dwords of codes) per step
          const uint32_t* kr = (const uint32_t*)(a.kp + phys * a.kps_blk + pos * a.kps_pos + h * a.kps_head);
          float sc[GQ];
#pragma unroll
          for (int q = 0; q < GQ; ++q) sc[q] = 0.f;
#pragma unroll 1
          for (int u = 0; u < D / 32; ++u) {
            uint32_t kw[BITS];
#pragma unroll
            for (int i = 0; i < BITS; ++i) kw[i] = kr[u * BITS + i];
            const float* qu = qh + u * 32;
#pragma unroll
            for (int d = 0; d < 32; ++d) {
              const uint32_t code = akv_stream_code<BITS>(d, [&](int o) { return (kw[o >> 2] >> (8 * (o & 3))) & 0xffu; });
              const float kv = cen[code];
#pragma unroll
              for (int q = 0; q < GQ; ++q) sc[q] = fmaf(qu[q * D + d], kv, sc[q]);
            }
          }
          const float knorm = a.kn[phys * a.kns_blk + pos * a.kns_pos + h * a.kns_head];
          const float vnorm = valid ? a.vn[phys * a.vns_blk + pos * a.vns_pos + h * a.vns_head] : 0.f;
          // ---- running softmax
#pragma unroll
          for (int q = 0; q < GQ; ++q) {
            const float sv = valid ? sc[q] * knorm * a.scale : -INFINITY;
            const float mt = akv_wave_max(sv);
            const float mn = fmaxf(m[q], mt);
            const float alpha = __expf(m[q] - mn);
            const float p = valid ? __expf(sv - mn) : 0.f;
            l[q] = l[q] * alpha + p;
#pragma unroll
            for (int i = 0; i < DPL; ++i) acc[q][i] *= alpha;
            m[q] = mn;
            p_lds[lane * GQ + q] = p * vnorm;
          }
          // ---- stage the V rows
          {
            const uint32_t* vr = (const uint32_t*)(a.vp + phys * a.vps_blk + pos * a.vps_pos + h * a.vps_head);
#pragma unroll
            for (int i = 0; i < ROWDW; ++i) v_lds[lane * VROW + i] = vr[i];
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          // ---- values: lanes <-> coordinates
          const int nt = min(64, t1 - c0);
          for (int tt = 0; tt < nt; ++tt) {
            const uint8_t* vb = (const uint8_t*)(v_lds + tt * VROW);
            float vv[DPL];
#pragma unroll
            for (int i = 0; i < DPL; ++i) {
              const uint32_t code = akv_stream_code<BITS>(lane * DPL + i, [&](int o) { return (uint32_t)vb[o]; });
              vv[i] = cen[code];
            }
#pragma unroll
            for (int q = 0; q < GQ; ++q) {
              const float pw = p_lds[tt * GQ + q];
#pragma unroll
              for (int i = 0; i < DPL; ++i) acc[q][i] = fmaf(pw, vv[i], acc[q][i]);
            }
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
        // ---- partial for this (workgroup, sequence, query heads)
#pragma unroll
        for (int q = 0; q < GQ; ++q) {
          const size_t slot = (size_t)(blockIdx.x + s) * a.QH + (h * gqa + qg + q);
          const float lsum = akv_wave_sum(l[q]);
#pragma unroll
          for (int i = 0; i < DPL; ++i) a.part_acc[slot * D + lane * DPL + i] = acc[q][i];
          if (lane == 0) { a.part_ml[slot * 2] = m[q]; a.part_ml[slot * 2 + 1] = lsum; }
        }
      }
    }
  }
}

// ----------------------------------------------------------------------------------
// host entry
// ----------------------------------------------------------------------------------
// MFMA path (akv_attn_mfma.hip)
size_t akv_attn_mfma_extra_bytes(int S, int KVH);
bool akv_attn_mfma_applicable(const akv_attn_args& a, int d, int bits);
int akv_attn_mfma_run(const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head, const float* PiT,
                      const akv_attn_args& a, int bits, const akv_attn_ws& ws, void* extra_ws, int grid, hipStream_t stream);

extern "C" size_t akv_paged_attn_workspace_bytes(int num_seqs, int num_q_heads, int d) {
  if (num_seqs < 0 || num_q_heads <= 0 || d <= 0) return 0;
  // the number of kv heads is not known here; it is at most the number of query heads
  return akv_attn_ws_layout(nullptr, num_seqs, num_q_heads, d, akv_attn_grid()).bytes +
         akv_attn_mfma_extra_bytes(num_seqs, num_q_heads);
}

static void* akv_static_scratch_of_current_device();   // null before the first akv_paged_attn_static call there

extern "C" int akv_paged_attn_status(const void* workspace, int* flags, void* stream_) {
  AKV_REQUIRE(flags != nullptr, "akv_paged_attn_status: null pointer");
  hipStream_t stream = (hipStream_t)stream_;
  if (workspace == nullptr) {
    // the built-in scratch array of akv_paged_attn_static on the current device
    workspace = akv_static_scratch_of_current_device();
    if (workspace == nullptr) { *flags = 0; return AKV_OK; }
  }
  uint32_t word = 0;
  AKV_HIP(hipMemcpyAsync(&word, (const char*)workspace + AKV_WS_LUT_BYTES, sizeof(word), hipMemcpyDeviceToHost, stream));
  AKV_HIP(hipStreamSynchronize(stream));
  *flags = (int)word;
  return AKV_OK;
}

template <int D, int BITS, int GQ>
static int akv_launch_attn_general_gq(const akv_attn_args& a, int grid, hipStream_t stream) {
  const size_t lds = akv_attn_gen_cfg<D, BITS, GQ>::lds_bytes(a.QH);
  if (lds > 160 * 1024)
    return akv_fail(AKV_ERR_UNSUPPORTED, "paged_attn: num_q_heads*head_dim too large for LDS (%zu bytes)", lds);
  AKV_HIP(hipFuncSetAttribute((const void*)akv_attn_general_kernel<D, BITS, GQ>,
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
  akv_profile_mark_begin(stream);
  akv_attn_general_kernel<D, BITS, GQ><<<grid, 64 * akv_attn_gen_waves<D>(), lds, stream>>>(a);
  akv_profile_mark_end(stream);
  AKV_LAUNCH_CHECK("akv_attn_general_kernel");
  return AKV_OK;
}

template <int D, int BITS>
static int akv_launch_attn_general(const akv_attn_args& a, int grid, hipStream_t stream) {
  const int gqa = a.QH / a.KVH;
  if (gqa % 4 == 0) return akv_launch_attn_general_gq<D, BITS, 4>(a, grid, stream);
  return akv_launch_attn_general_gq<D, BITS, 1>(a, grid, stream);
}

template <int D>
static int akv_launch_reduce(int odt, const akv_attn_args& a, const float* Pi, const uint4* bop, int G, void* out,
                             int64_t os_seq, int64_t os_head, const uint32_t* status, const int32_t* seqw, hipStream_t stream) {
  // at most three workgroups per CU (what its registers admit at once); a workgroup loops over its items
  const int items = a.S * ((a.QH + 3) / 4);
  const int cus = akv_cached_cu_count();
  const int grid = items < 3 * (cus > 0 ? cus : 256) ? items : 3 * (cus > 0 ? cus : 256);
  switch (odt) {
    case AKV_F16: akv_attn_reduce_kernel<D, AKV_F16><<<grid, 256, 0, stream>>>(a.prefix, a.part_acc, a.part_ml, Pi, bop, a.S, a.QH, G, out, os_seq, os_head, status, seqw); break;
    case AKV_BF16: akv_attn_reduce_kernel<D, AKV_BF16><<<grid, 256, 0, stream>>>(a.prefix, a.part_acc, a.part_ml, Pi, bop, a.S, a.QH, G, out, os_seq, os_head, status, seqw); break;
    default: akv_attn_reduce_kernel<D, AKV_F32><<<grid, 256, 0, stream>>>(a.prefix, a.part_acc, a.part_ml, Pi, bop, a.S, a.QH, G, out, os_seq, os_head, status, seqw); break;
  }
  AKV_LAUNCH_CHECK("akv_attn_reduce_kernel");
  return AKV_OK;
}

static int akv_paged_attn_impl(
    const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
    const uint8_t* k_packed, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
    const float* k_norms, int64_t kns_blk, int64_t kns_pos, int64_t kns_head,
    const uint8_t* v_packed, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
    const float* v_norms, int64_t vns_blk, int64_t vns_pos, int64_t vns_head,
    const void* block_tables, int bt_itype, int64_t bt_stride,
    const void* context_lens, int cl_itype,
    const void* rot_prep, const float* centroids, int bits,
    void* out, int out_dtype, int64_t os_seq, int64_t os_head,
    int num_seqs, int num_q_heads, int num_kv_heads, int d,
    int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
    void* workspace, size_t workspace_bytes, void* stream_) {
  hipStream_t stream = (hipStream_t)stream_;
  AKV_REQUIRE(num_seqs >= 0 && num_q_heads > 0 && num_kv_heads > 0, "akv_paged_attn: bad head/seq counts");
  AKV_REQUIRE(num_blocks > 0 || max_blocks_per_seq == 0, "akv_paged_attn: num_blocks=%lld with a non-empty block table", (long long)num_blocks);
  AKV_REQUIRE(num_q_heads % num_kv_heads == 0, "akv_paged_attn: num_q_heads %% num_kv_heads != 0");
  AKV_REQUIRE(akv_valid_dtype(q_dtype) && akv_valid_dtype(out_dtype), "akv_paged_attn: bad dtype");
  AKV_REQUIRE(akv_valid_itype(bt_itype) && akv_valid_itype(cl_itype), "akv_paged_attn: bad index type");
  AKV_REQUIRE(block_size > 0 && max_blocks_per_seq >= 0, "akv_paged_attn: bad block_size / table width");
  AKV_REQUIRE(bits >= 2 && bits <= 4, "akv_paged_attn: bits=%d not in {2,3,4}", bits);
  if (!(d == 64 || d == 128 || d == 256 || d == 512))
    return akv_fail(AKV_ERR_UNSUPPORTED, "akv_paged_attn: head_dim=%d not in {64,128,256,512}", d);
  if (num_seqs == 0) return AKV_OK;
  AKV_REQUIRE(query && out && rot_prep && centroids && context_lens, "akv_paged_attn: null pointer");
  AKV_REQUIRE(max_blocks_per_seq == 0 || (k_packed && k_norms && v_packed && v_norms && block_tables),
              "akv_paged_attn: null cache pointer");
  AKV_REQUIRE((((uintptr_t)k_packed | (uintptr_t)v_packed | (uintptr_t)kps_blk | (uintptr_t)kps_pos |
                (uintptr_t)kps_head | (uintptr_t)vps_blk | (uintptr_t)vps_pos | (uintptr_t)vps_head) & 3) == 0,
              "akv_paged_attn: packed rows must be 4-byte aligned");
  const int G = akv_attn_grid();
  AKV_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 255) == 0, "akv_paged_attn: workspace null or not 256-byte aligned");
  akv_attn_ws ws = akv_attn_ws_layout(workspace, num_seqs, num_q_heads, d, G);
  if (workspace_bytes < ws.bytes)
    return akv_fail(AKV_ERR_WORKSPACE, "akv_paged_attn: workspace %zu < %zu bytes", workspace_bytes, ws.bytes);

  if (workspace_bytes < ws.bytes + akv_attn_mfma_extra_bytes(num_seqs, num_q_heads))
    return akv_fail(AKV_ERR_WORKSPACE, "akv_paged_attn: workspace %zu < %zu bytes", workspace_bytes,
                    ws.bytes + akv_attn_mfma_extra_bytes(num_seqs, num_q_heads));
  const float* Pi = (const float*)rot_prep;
  const float* PiT = Pi + (size_t)d * d;

  akv_attn_args a;
  a.kp = k_packed; a.kps_blk = kps_blk; a.kps_pos = kps_pos; a.kps_head = kps_head;
  a.kn = k_norms; a.kns_blk = kns_blk; a.kns_pos = kns_pos; a.kns_head = kns_head;
  a.vp = v_packed; a.vps_blk = vps_blk; a.vps_pos = vps_pos; a.vps_head = vps_head;
  a.vn = v_norms; a.vns_blk = vns_blk; a.vns_pos = vns_pos; a.vns_head = vns_head;
  a.block_tables = block_tables; a.bt_itype = bt_itype; a.bt_stride = bt_stride;
  a.context_lens = context_lens; a.cl_itype = cl_itype;
  a.centroids = centroids;
  a.S = num_seqs; a.QH = num_q_heads; a.KVH = num_kv_heads; a.block_size = block_size;
  a.max_blocks_per_seq = max_blocks_per_seq; a.num_blocks = num_blocks; a.scale = scale;
  a.prefix = ws.prefix; a.qrot = ws.qrot; a.part_acc = ws.part_acc; a.part_ml = ws.part_ml;
  a.hgroup = 1;

  int rc;
  int Gused = G;
  const int32_t* seqw = nullptr;      // set by the matrix-core path, whose prologue cuts the block axis itself
  if (akv_attn_mfma_applicable(a, d, bits)) {
    seqw = ws.seqw;
    Gused = G / AKV_ATTN_WG_PER_CU;   // one 8-wavefront workgroup per CU (64 KiB table, up to 256 VGPRs)
    rc = akv_attn_mfma_run(query, q_dtype, qs_seq, qs_head, PiT, a, bits, ws, (char*)workspace + ws.bytes, Gused, stream);
  } else {
    const int pgrid = num_seqs * num_q_heads + 1;
#define AKV_PRO(DT) akv_attn_prologue_kernel<DT><<<pgrid, 256, 0, stream>>>(query, qs_seq, qs_head, PiT, num_seqs, num_q_heads, d, context_lens, cl_itype, block_size, max_blocks_per_seq, ws.prefix, ws.qrot, ws.status)
    if (q_dtype == AKV_F16) AKV_PRO(AKV_F16); else if (q_dtype == AKV_BF16) AKV_PRO(AKV_BF16); else AKV_PRO(AKV_F32);
#undef AKV_PRO
    AKV_LAUNCH_CHECK("akv_attn_prologue_kernel");
    rc = AKV_ERR_UNSUPPORTED;
#define AKV_CASE(DD, BB) if (d == DD && bits == BB) rc = akv_launch_attn_general<DD, BB>(a, G, stream);
    AKV_CASE(64, 2) AKV_CASE(64, 3) AKV_CASE(64, 4)
    AKV_CASE(128, 2) AKV_CASE(128, 3) AKV_CASE(128, 4)
    AKV_CASE(256, 2) AKV_CASE(256, 3) AKV_CASE(256, 4)
    AKV_CASE(512, 2) AKV_CASE(512, 3) AKV_CASE(512, 4)
#undef AKV_CASE
  }
  if (rc) return rc;
  if (d == 64) return akv_launch_reduce<64>(out_dtype, a, Pi, nullptr, Gused, out, os_seq, os_head, ws.status, seqw, stream);
  if (d == 128) return akv_launch_reduce<128>(out_dtype, a, Pi, (const uint4*)((const char*)rot_prep + AKV_PREP_DECODE_OFFSET(128)), Gused, out, os_seq, os_head, ws.status, seqw, stream);
  if (d == 256) return akv_launch_reduce<256>(out_dtype, a, Pi, nullptr, Gused, out, os_seq, os_head, ws.status, seqw, stream);
  return akv_launch_reduce<512>(out_dtype, a, Pi, nullptr, Gused, out, os_seq, os_head, ws.status, seqw, stream);
}

extern "C" int akv_paged_attn(
    const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
    const uint8_t* k_packed, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
    const float* k_norms, int64_t kns_blk, int64_t kns_pos, int64_t kns_head,
    const uint8_t* v_packed, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
    const float* v_norms, int64_t vns_blk, int64_t vns_pos, int64_t vns_head,
    const void* block_tables, int bt_itype, int64_t bt_stride,
    const void* context_lens, int cl_itype,
    const void* rot_prep, const float* centroids, int bits,
    void* out, int out_dtype, int64_t os_seq, int64_t os_head,
    int num_seqs, int num_q_heads, int num_kv_heads, int d,
    int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale,
    void* workspace, size_t workspace_bytes, void* stream) {
  return akv_paged_attn_impl(query, q_dtype, qs_seq, qs_head, k_packed, kps_blk, kps_pos, kps_head,
                             k_norms, kns_blk, kns_pos, kns_head, v_packed, vps_blk, vps_pos, vps_head,
                             v_norms, vns_blk, vns_pos, vns_head, block_tables, bt_itype, bt_stride,
                             context_lens, cl_itype, rot_prep, centroids, bits, out, out_dtype, os_seq, os_head,
                             num_seqs, num_q_heads, num_kv_heads, d, block_size, num_blocks, max_blocks_per_seq,
                             scale, workspace, workspace_bytes, stream);
}

// ----------------------------------------------------------------------------------
// The same call for callers that cannot bring a workspace of their own and cannot allocate one
// (code under HIP-graph capture, serving loops and harnesses that forbid allocation): the rotated
// queries, the split partials and the cached tables live in a fixed array inside the library's
// device image.  The array's name is a host-side stand-in, not a device address: its address on a
// device is asked for once per device (hipGetSymbolAddress, with that device current) and only that
// pointer is ever handed to kernels.  Every call on a GPU shares that GPU's array: the kernels
// rewrite every word they read (the prologue clears the status word, rebuilds the prefix and the
// query operands; the table block is validated by its tag), and calls that overlap on one GPU race.
// ----------------------------------------------------------------------------------
#define AKV_STATIC_SCRATCH_BYTES ((size_t)32 << 20)
#define AKV_STATIC_MAX_DEVICES 64
static __device__ __align__(256) unsigned char akv_attn_scratch[AKV_STATIC_SCRATCH_BYTES];
static void* g_attn_scratch_ptr[AKV_STATIC_MAX_DEVICES];

static void* akv_static_scratch_of_current_device() {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= AKV_STATIC_MAX_DEVICES) return nullptr;
  return __atomic_load_n(&g_attn_scratch_ptr[dev], __ATOMIC_ACQUIRE);
}

extern "C" size_t akv_paged_attn_static_scratch_bytes(void) { return AKV_STATIC_SCRATCH_BYTES; }

extern "C" int akv_paged_attn_static(
    const void* query, int q_dtype, int64_t qs_seq, int64_t qs_head,
    const uint8_t* k_packed, int64_t kps_blk, int64_t kps_pos, int64_t kps_head,
    const float* k_norms, int64_t kns_blk, int64_t kns_pos, int64_t kns_head,
    const uint8_t* v_packed, int64_t vps_blk, int64_t vps_pos, int64_t vps_head,
    const float* v_norms, int64_t vns_blk, int64_t vns_pos, int64_t vns_head,
    const void* block_tables, int bt_itype, int64_t bt_stride,
    const void* context_lens, int cl_itype,
    const void* rot_prep, const float* centroids, int bits,
    void* out, int out_dtype, int64_t os_seq, int64_t os_head,
    int num_seqs, int num_q_heads, int num_kv_heads, int d,
    int block_size, int64_t num_blocks, int64_t max_blocks_per_seq, float scale, void* stream) {
  AKV_REQUIRE(num_seqs >= 0 && num_q_heads > 0 && d > 0, "akv_paged_attn_static: bad head/seq counts");
  const size_t need = akv_paged_attn_workspace_bytes(num_seqs, num_q_heads, d);
  if (need > AKV_STATIC_SCRATCH_BYTES)
    return akv_fail(AKV_ERR_WORKSPACE,
                    "akv_paged_attn_static: %d sequences x %d query heads need %zu bytes of scratch, the built-in "
                    "array holds %zu; use akv_paged_attn with a workspace of your own",
                    num_seqs, num_q_heads, need, (size_t)AKV_STATIC_SCRATCH_BYTES);
  int dev = -1;
  AKV_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= AKV_STATIC_MAX_DEVICES)
    return akv_fail(AKV_ERR_UNSUPPORTED, "akv_paged_attn_static: device index %d beyond %d", dev, AKV_STATIC_MAX_DEVICES);
  void* ptr = __atomic_load_n(&g_attn_scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (ptr == nullptr) {
    // first call on this device (two threads racing here both obtain the same address)
    AKV_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(akv_attn_scratch)));
    if (ptr == nullptr || ((uintptr_t)ptr & 255) != 0)
      return akv_fail(AKV_ERR_HIP, "akv_paged_attn_static: built-in scratch array has no usable device address");
    __atomic_store_n(&g_attn_scratch_ptr[dev], ptr, __ATOMIC_RELEASE);
  }
  return akv_paged_attn_impl(query, q_dtype, qs_seq, qs_head, k_packed, kps_blk, kps_pos, kps_head,
                             k_norms, kns_blk, kns_pos, kns_head, v_packed, vps_blk, vps_pos, vps_head,
                             v_norms, vns_blk, vns_pos, vns_head, block_tables, bt_itype, bt_stride,
                             context_lens, cl_itype, rot_prep, centroids, bits, out, out_dtype, os_seq, os_head,
                             num_seqs, num_q_heads, num_kv_heads, d, block_size, num_blocks, max_blocks_per_seq,
                             scale, ptr, AKV_STATIC_SCRATCH_BYTES, stream);
}
