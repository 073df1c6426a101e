// GAAC tile format for gfx950 (wave64, MFMA fragment order) and the per-unit decoder shared by every kernel.
//
// Format semantics (element split, channel permutation, 8-element groups, tier rule, 3-bit codes, tag words,
// escape stream) follow /root/reference/gaac/codec.py:133-218.  Only the BYTE ORDER of the sign/mantissa and
// code bytes inside a 16-token tile is different: it is the operand order of the gfx950 MFMA instructions the
// attention kernel issues, laid out so that every wave-wide load is one contiguous 1 KiB / 256 B segment.
//
// A tile (16 tokens x 128 stored positions) is owned by one wave64.  Lane l = a + 16*q owns four UNITS
// (a unit = one 8-element group of one token: 8 sign/mantissa bytes, one 24-bit code word, one 2-bit tag):
//   K tile: a = token, q = group quad       -> unit u = (token a,      group 4q+u)
//   V tile: a = group, q = token quad       -> unit u = (token 4q+u,   group a)
// Native byte order of a tile:
//   sign/mantissa (2048 B): byte 1024*j + 16*l + 8*v + i  = element i of unit 2j+v of lane l   (j,v in {0,1})
//   codes (768 B):          byte 256*k + 4*l + b          = byte 4k+b of the lane's 12 code bytes (unit u -> bytes 3u..3u+2)
// Tag words (16 x u32 per tile) and escape bytes are stored per LINE a = l & 15 of the tile: word a holds the 2-bit tags
// of the 16 units of line a, unit (a, j) at bits 2j (lane a+16q owns bits 8q..8q+7); the tile's escape bytes follow line
// order (a ascending, j ascending; 1 byte per 4-bit group, 5 bytes per raw group).  For K a line is a token row and j the
// group, which IS the reference order; for V a line is a group and j the token, i.e. the 16 x 16 tag matrix and the
// escape order of a V tile are the transpose of the reference's.  Tile offsets and per-tile byte counts are unaffected.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gaac {

typedef uint32_t u32;
typedef uint64_t u64;
typedef uint16_t u16;

constexpr int D = 128;        // head dim
constexpr int T = 16;         // tokens per tile
constexpr int GS = 8;         // elements per group
constexpr int NG = 16;        // groups per token row
constexpr int CB = 48;        // code bytes per token row
constexpr int TILE_SM = T * D;      // 2048
constexpr int TILE_CD = T * CB;     // 768
constexpr int TILE_MAX_ESC = T * NG * 5;   // 1280
constexpr int KIND_K = 0, KIND_V = 1;

typedef __attribute__((ext_vector_type(4))) u32 u32x4;
typedef __attribute__((ext_vector_type(2))) u32 u32x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// stored position -> channel (codec.py:29-45)
__host__ __device__ constexpr int chan_k(int pos) { return 16 * ((pos >> 2) & 7) + 2 * (pos >> 5) + (pos & 1) + 8 * ((pos >> 1) & 1); }
__host__ __device__ constexpr int chan_v(int pos) { return 8 * (pos & 15) + (pos >> 4); }
template <int KIND> __host__ __device__ constexpr int chan_of(int pos) { return KIND == KIND_K ? chan_k(pos) : chan_v(pos); }

// unit u of lane (a, q) -> (token in tile, group)
template <int KIND> __device__ __forceinline__ int unit_token(int a, int q, int u) { return KIND == KIND_K ? a : 4 * q + u; }
template <int KIND> __device__ __forceinline__ int unit_group(int a, int q, int u) { return KIND == KIND_K ? 4 * q + u : a; }

// escape bytes of the groups below bit position `bits` of a tag word: 4-bit group -> 1 byte, raw group (both bits) -> 5 bytes
__device__ __forceinline__ int esc_bytes(u32 fl) { return __popc(fl & 0x55555555u) + 4 * __popc(fl & 0xAAAAAAAAu); }
__device__ __forceinline__ int esc_prefix(u32 fl, int bits) { return esc_bytes(__builtin_amdgcn_ubfe(fl, 0, bits)); }
__device__ __forceinline__ int tag_size(u32 t) { return (int)((t & 1u) + 2u * (t & 2u)); }    // 0 -> 0, 1 -> 1, 3 -> 5

__device__ __forceinline__ u32 dpp_row_shr(u32 v, int n) {   // lanes shifted in from outside the 16-lane row read 0
  switch (n) {
    case 1: return __builtin_amdgcn_update_dpp(0u, v, 0x111, 0xF, 0xF, true);
    case 2: return __builtin_amdgcn_update_dpp(0u, v, 0x112, 0xF, 0xF, true);
    case 4: return __builtin_amdgcn_update_dpp(0u, v, 0x114, 0xF, 0xF, true);
    default: return __builtin_amdgcn_update_dpp(0u, v, 0x118, 0xF, 0xF, true);
  }
}
// inclusive prefix sum over the 16 lanes of each DPP row
__device__ __forceinline__ u32 row_scan16(u32 v) {
  v += dpp_row_shr(v, 1); v += dpp_row_shr(v, 2); v += dpp_row_shr(v, 4); v += dpp_row_shr(v, 8);
  return v;
}
// all-reduce across the four 16-lane rows at fixed column (lanes c, c+16, c+32, c+48)
__device__ __forceinline__ float quad_rows_max(float v) {
  u32 x = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  x = __float_as_uint(v);
  auto s = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  return fmaxf(__uint_as_float(s[0]), __uint_as_float(s[1]));
}
__device__ __forceinline__ float quad_rows_sum(float v) {
  u32 x = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  x = __float_as_uint(v);
  auto s = __builtin_amdgcn_permlane16_swap(x, x, false, false);
  return __uint_as_float(s[0]) + __uint_as_float(s[1]);
}

// all-reduce over the 64 lanes of the wave without LDS traffic: four DPP steps inside each 16-lane row, then across the rows
#define GAAC_ROW16_REDUCE(v, OP)                                                   \
  v = OP(v, __uint_as_float((u32)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0xB1, 0xF, 0xF, true)));  /* quad_perm [1,0,3,2] */ \
  v = OP(v, __uint_as_float((u32)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x4E, 0xF, 0xF, true)));  /* quad_perm [2,3,0,1] */ \
  v = OP(v, __uint_as_float((u32)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x141, 0xF, 0xF, true))); /* row_half_mirror */      \
  v = OP(v, __uint_as_float((u32)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), 0x140, 0xF, 0xF, true)))  /* row_mirror */
__device__ __forceinline__ float gaac_addf(float a, float b) { return a + b; }
__device__ __forceinline__ float wave_max(float v) { GAAC_ROW16_REDUCE(v, fmaxf); return quad_rows_max(v); }
__device__ __forceinline__ float wave_sum(float v) { GAAC_ROW16_REDUCE(v, gaac_addf); return quad_rows_sum(v); }

// ---- exponent-base words ------------------------------------------------------------------------------------------
// Word p of a group pairs elements p (low half) and p+4 (high half): base << 7 | base' << 23 sits on the exponent fields.
template <int KIND>
__device__ __forceinline__ void load_base_words(const uint8_t* __restrict__ base_row, int group, u32* w /*[4]*/) {
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    u32 lo = base_row[chan_of<KIND>(8 * group + p)], hi = base_row[chan_of<KIND>(8 * group + p + 4)];
    w[p] = (lo << 7) | (hi << 23);
  }
}

// ---- the unit decoder ---------------------------------------------------------------------------------------------
// slo/shi: sign/mantissa bytes of elements 0-3 / 4-7;  g24: the group's code word (code i at bits 3i);  tag: 0 | 1 | 3;
// eb: the group's escape byte when tag == 1, else 0;  esc: address of the group's escape bytes (read only when tag == 3).
// out[p] = bf16x2 (element p, element p+4), p = 0..3: bit-exact BF16.
constexpr u32 EXP_MASK2 = 0x7F807F80u;
__device__ __forceinline__ void decode_unit(u32 slo, u32 shi, u32 g24, u32 tag, u32 eb, const uint8_t* __restrict__ esc,
                                            const u32* __restrict__ b3w, const u32* __restrict__ b4w, u32* __restrict__ out) {
  const u32 cw = (g24 & 0xFFFu) | ((g24 << 4) & 0x0FFF0000u);      // low-half codes at bits 3p, high-half codes at bits 16+3p
  const u32 xw = eb | (eb << 12);                                   // 4th bits: element p at bit p, element p+4 at bit 16+p
  const bool t0 = tag == 0u;
  u32 sw[4], cc[4];
  sw[0] = __builtin_amdgcn_perm(shi, slo, 0x04040000u);
  sw[1] = __builtin_amdgcn_perm(shi, slo, 0x05050101u);
  sw[2] = __builtin_amdgcn_perm(shi, slo, 0x06060202u);
  sw[3] = __builtin_amdgcn_perm(shi, slo, 0x07070303u);
  cc[0] = (cw << 7) & 0x03800380u; cc[1] = (cw << 4) & 0x03800380u; cc[2] = (cw << 1) & 0x03800380u; cc[3] = (cw >> 2) & 0x03800380u;
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    u32 x = (xw << (10 - p)) & 0x04000400u;
    u32 e2 = cc[p] + (t0 ? b3w[p] : b4w[p]) + x;
    out[p] = (e2 & EXP_MASK2) | (sw[p] & ~EXP_MASK2);
  }
  if (tag == 3u) {      // raw group (about 0.2 % of groups): 5 bytes = 8 x 5 high exponent bits, little endian
    u64 hi = (u64)esc[0] | ((u64)esc[1] << 8) | ((u64)esc[2] << 16) | ((u64)esc[3] << 24) | ((u64)esc[4] << 32);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      u32 e2 = cc[p] | ((u32)((hi >> (5 * p)) & 31u) << 10) | ((u32)((hi >> (5 * p + 20)) & 31u) << 26);
      out[p] = (e2 & EXP_MASK2) | (sw[p] & ~EXP_MASK2);
    }
  }
}

// code word of unit u out of the lane's three code dwords
__device__ __forceinline__ u32 unit_code_word(u32 c0, u32 c1, u32 c2, int u) {
  switch (u) {
    case 0: return c0;
    case 1: return __builtin_amdgcn_alignbit(c1, c0, 24);
    case 2: return __builtin_amdgcn_alignbit(c2, c1, 16);
    default: return c2 >> 8;
  }
}

// ---- per-lane tile payload ----------------------------------------------------------------------------------------
struct Payload {          // one lane's share of a tile: 32 sign/mantissa bytes + 12 code bytes
  u32x4 s0, s1;           // units 0,1 | units 2,3
  u32 c0, c1, c2;
};
__device__ __forceinline__ void load_payload(const uint8_t* __restrict__ sm_tile, const uint8_t* __restrict__ cd_tile, int lane, Payload& P) {
  // streamed once: non-temporal loads (measured on a plain read stream: 8 % more bandwidth than loads that allocate in the caches)
  P.s0 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sm_tile + 16 * lane));
  P.s1 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(sm_tile + 1024 + 16 * lane));
  P.c0 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(cd_tile + 4 * lane));
  P.c1 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(cd_tile + 256 + 4 * lane));
  P.c2 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(cd_tile + 512 + 4 * lane));
}
__device__ __forceinline__ void unit_sm(const Payload& P, int u, u32& slo, u32& shi) {
  switch (u) {
    case 0: slo = P.s0[0]; shi = P.s0[1]; break;
    case 1: slo = P.s0[2]; shi = P.s0[3]; break;
    case 2: slo = P.s1[0]; shi = P.s1[1]; break;
    default: slo = P.s1[2]; shi = P.s1[3]; break;
  }
}

// unaligned little-endian loads from the escape stream (the stream is padded by 8 bytes at the end)
__device__ __forceinline__ u32x2 load_u32x2_unaligned(const uint8_t* p) { u32x2 v; __builtin_memcpy(&v, p, 8); return v; }
__device__ __forceinline__ u64 load_u64_unaligned(const uint8_t* p) {
  u32x2 v; __builtin_memcpy(&v, p, 8); return (u64)v[0] | ((u64)v[1] << 32);
}

}  // namespace gaac
