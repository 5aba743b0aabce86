// Spreading 3-bit and 2-bit code streams to one code per nibble (two codes per byte), the form the
// byte-indexed lookup tables of the matrix-core kernels take, and the coordinate order that results.
#ifndef AKV_NIBBLE_H
#define AKV_NIBBLE_H
#include <stdint.h>
#include <hip/hip_runtime.h>

// Code order after spreading.  Row side (K rows of attention, rows of decode): spread dword st (0..3)
// of lane g, byte b, nibble `lo` (0 = high nibble) -> coordinate inside the lane's 32.  V side of
// attention: M-tile n of the value product <-> coordinate inside the lane's 8.
template <int BITS>
__host__ __device__ constexpr int mf_kcoord(int st, int b, int lo) {
  if (BITS == 4) return 8 * st + 2 * b + lo;
  if (BITS == 2) return 16 * (st >> 1) + 4 * b + ((st & 1) ? 2 * lo : 1 + 2 * lo);   // W & 0x33.. | (W >> 2) & 0x33..
  // 3-bit: bytes (c6,c7) (c3,c5) (c1,c2) (c0,c4) of each group of eight codes (see mf_spread3)
  constexpr int hi3[4] = {6, 3, 1, 0}, lo3[4] = {7, 5, 2, 4};
  return 8 * st + (lo ? lo3[b] : hi3[b]);
}
template <int BITS>
__host__ __device__ constexpr int mf_vtile_of_coord(int k) {
  if (BITS == 4) return k;
  if (BITS == 2) { constexpr int inv[8] = {2, 3, 0, 1, 6, 7, 4, 5}; return inv[k]; }
  constexpr int inv[8] = {6, 4, 5, 2, 7, 3, 0, 1};
  return inv[k];
}
// eight 3-bit codes c0..c7 (c0 in bits 23:21 of w) -> nibbles [c7 c6 c5 c3 c2 c1 c4 c0] from bit 0 up
__device__ __forceinline__ uint32_t mf_spread3(uint32_t w) {
  uint32_t t = w & 0x7007u;
  t = ((w << 1) & 0x70070u) | t;
  t = ((w << 2) & 0x700700u) | t;
  t = ((w << 15) & 0x07000000u) | t;
  t = ((w << 7) & 0x70000000u) | t;
  return t;
}
// eight 2-bit codes in a halfword (byte 0 = c0..c3 from the top bits) -> bytes (c2,c3) (c0,c1) (c6,c7) (c4,c5)
__device__ __forceinline__ uint32_t mf_spread2(uint32_t h) {
  uint32_t t = (h | (h << 8)) & 0x00FF00FFu;
  t = (t | (t << 4)) & 0x0F0F0F0Fu;
  t = (t | (t << 2)) & 0x33333333u;
  return t;
}

// the lane's quarter of a packed row (32 codes: 16 / 12 / 8 bytes in w[0..3] / w[0..2] / w[0..1]) as four
// nibble dwords; dword st, byte b, nibble lo holds coordinate mf_kcoord<BITS>(st, b, lo) of the 32
template <int BITS>
__device__ __forceinline__ void mf_spread_row(const uint32_t (&w)[4], uint32_t (&kw)[4]) {
  if constexpr (BITS == 4) {
    kw[0] = w[0]; kw[1] = w[1]; kw[2] = w[2]; kw[3] = w[3];
  } else if constexpr (BITS == 2) {
    kw[0] = w[0] & 0x33333333u; kw[1] = (w[0] >> 2) & 0x33333333u;
    kw[2] = w[1] & 0x33333333u; kw[3] = (w[1] >> 2) & 0x33333333u;
  } else {
    // group q = bytes 3q .. 3q+2 of the twelve, as one big-endian 24-bit word
    kw[0] = mf_spread3(__builtin_amdgcn_perm(w[0], w[0], 0x0c000102u));
    kw[1] = mf_spread3(__builtin_amdgcn_perm(w[1], w[0], 0x0c030405u));
    kw[2] = mf_spread3(__builtin_amdgcn_perm(w[2], w[1], 0x0c020304u));
    kw[3] = mf_spread3(__builtin_amdgcn_perm(w[2], w[2], 0x0c010203u));
  }
}
#endif  // AKV_NIBBLE_H
