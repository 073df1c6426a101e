// Wave-level tile encoder and tile metadata helpers (one wave64 = one 16-token tile), shared by the page encoder,
// the cache append kernel and the paged store.  Tier rule, code words, tag words and escape bytes follow
// /root/reference/gaac/codec.py:138-172 and /root/reference/gaac/encoder.py:30-66; byte placement is the native one
// described in gaac_core.h.
#pragma once
#include "gaac_core.h"

namespace gaac {

// LDS scratch of one encoding wave
constexpr int XROW = D + 8;     // staged row stride in elements: 16 padding bytes spread the sixteen rows of a column over the banks
struct EncodeLds {
  u16 x[T * XROW];     // the tile's BF16 bit patterns, token-major, natural channel order (rows >= nvalid are zero)
  uint8_t b3[D], b4[D];
  u32 tags[T];
  int rowoff[T + 1];   // exclusive prefix of per-row escape bytes; [16] = tile total
};

// 16 rows of 128 BF16 (row r at src + r*row_stride elements): lane's four 16-byte pieces; rows >= nvalid read as zero.
struct RowRegs { u32x4 v[4]; };
__device__ __forceinline__ void load_rows(RowRegs& R, const u16* __restrict__ src, long row_stride, int nvalid, int lane) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    R.v[k] = u32x4{0u, 0u, 0u, 0u};
    if (row < nvalid) R.v[k] = *reinterpret_cast<const u32x4*>(src + (long)row * row_stride + c16 * 8);
  }
}
__device__ __forceinline__ void store_rows(EncodeLds& L, const RowRegs& R, int lane) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    *reinterpret_cast<u32x4*>(&L.x[row * XROW + c16 * 8]) = R.v[k];
  }
}
// Stage 16 rows into lds.x
__device__ __forceinline__ void stage_rows(EncodeLds& L, const u16* __restrict__ src, long row_stride, int nvalid, int lane) {
  RowRegs R;
  load_rows(R, src, row_stride, nvalid, lane);
  store_rows(L, R, lane);
}
__device__ __forceinline__ void stage_bases(EncodeLds& L, const uint8_t* __restrict__ b3row, const uint8_t* __restrict__ b4row, int lane) {
  if (lane < 32) reinterpret_cast<u32*>(L.b3)[lane] = reinterpret_cast<const u32*>(b3row)[lane];
  else reinterpret_cast<u32*>(L.b4)[lane - 32] = reinterpret_cast<const u32*>(b4row)[lane - 32];
  if (lane < T) L.tags[lane] = 0u;
}

// Orders the LDS traffic of ONE wave (LDS operations of a wave complete in program order; the fences only stop the compiler from
// moving them): what any lane wrote before is visible to every lane of the same wave after.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront"); __builtin_amdgcn_wave_barrier(); __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// The encoder works on 32-bit words that hold elements i and i+4 of a unit in their 16-bit halves (the decoder's word order), two
// elements per VALU operation.
struct BaseRegs { u32 b3[4][4], b4[4][4]; };      // [unit][i]: base of element i | base of element i+4 << 16
template <int KIND>
__device__ __forceinline__ void load_base_regs(const EncodeLds& L, int a, int q, BaseRegs& B) {
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int grp = unit_group<KIND>(a, q, u);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int c0 = chan_of<KIND>(8 * grp + i), c1 = chan_of<KIND>(8 * grp + i + 4);
      B.b3[u][i] = (u32)L.b3[c0] | ((u32)L.b3[c1] << 16);
      B.b4[u][i] = (u32)L.b4[c0] | ((u32)L.b4[c1] << 16);
    }
  }
}
// the four data words of unit u of lane (a, q)
template <int KIND>
__device__ __forceinline__ void unit_data_words(const EncodeLds& L, int a, int q, int u, u32* __restrict__ W) {
  if (KIND == KIND_K) {
    // elements (2m, 2m+1) are the adjacent channels 32u + 2q + 8m (+1): four aligned words, re-paired to (i, i+4)
    const u32* xr = reinterpret_cast<const u32*>(&L.x[a * XROW + 32 * u + 2 * q]);
    const u32 r0 = xr[0], r1 = xr[4], r2 = xr[8], r3 = xr[12];
    W[0] = __builtin_amdgcn_perm(r2, r0, 0x05040100u); W[1] = __builtin_amdgcn_perm(r2, r0, 0x07060302u);
    W[2] = __builtin_amdgcn_perm(r3, r1, 0x05040100u); W[3] = __builtin_amdgcn_perm(r3, r1, 0x07060302u);
  } else {
    // element i is channel 64 (a & 1) + (a >> 1) + 8 i of token 4q + u
    const u16* xr = &L.x[(4 * q + u) * XROW + 64 * (a & 1) + (a >> 1)];
#pragma unroll
    for (int i = 0; i < 4; ++i) W[i] = (u32)xr[8 * i] | ((u32)xr[8 * i + 32] << 16);
  }
}
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32 pk_sub_u16(u32 x, u32 y) {
  return __builtin_bit_cast(u32, (u16x2_t)(__builtin_bit_cast(u16x2_t, x) - __builtin_bit_cast(u16x2_t, y)));
}

// Encodes the tile staged in L (after a barrier).  Writes the native sign/mantissa and code bytes, the 16 tag words (one per line) and
// the escape bytes (at esc_dst + offset-in-tile; nullptr = count only).  Returns the tile's escape byte count (all lanes).
// Must be called by all 64 lanes of the wave that owns L; it synchronises that wave only.  B: load_base_regs of the same L.
template <int KIND>
__device__ __forceinline__ int encode_staged_tile(EncodeLds& L, const BaseRegs& B, int nvalid, int lane, uint8_t* __restrict__ sm_tile,
                                                  uint8_t* __restrict__ cd_tile, int* __restrict__ flags_tile,
                                                  uint8_t* __restrict__ esc_dst) {
  const int a = lane & 15, q = lane >> 4;
  u32 slo[4], shi[4], g24[4], tag[4], eb[4], ew[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 W[4], d3[4], d4[4];
    unit_data_words<KIND>(L, a, q, u, W);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ew[u][i] = (W[i] >> 7) & 0x00FF00FFu;                      // exponents
      d3[i] = pk_sub_u16(ew[u][i], B.b3[u][i]); d4[i] = pk_sub_u16(ew[u][i], B.b4[u][i]);      // negative differences wrap to >= 0xFF01
    }
    // tier rule (codec.py:144-150): all eight differences in 0..7, else all in 0..15, else raw
    const bool fit3 = ((d3[0] | d3[1] | d3[2] | d3[3]) & 0xFFF8FFF8u) == 0u, fit4 = ((d4[0] | d4[1] | d4[2] | d4[3]) & 0xFFF0FFF0u) == 0u;
    const bool valid = unit_token<KIND>(a, q, u) < nvalid;       // padded rows: tier 0, code 0, sign/mantissa 0
    u32 cacc = 0u, xacc = 0u, sb[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const u32 c = fit3 ? d3[i] : (fit4 ? d4[i] : ew[u][i]);
      cacc |= (c & 0x00070007u) << (3 * i);                       // code of element i at bits 3i, of element i+4 at 16 + 3i
      xacc |= (d4[i] & 0x00080008u) << i;                         // 4th code bit of element i at bit 3 + i, of i+4 at 19 + i
      sb[i] = ((W[i] >> 8) & 0x00800080u) | (W[i] & 0x007F007Fu); // sign/mantissa bytes at bits 0..7 and 16..23
    }
    const u32 p01 = __builtin_amdgcn_perm(sb[1], sb[0], 0x06020400u), p23 = __builtin_amdgcn_perm(sb[3], sb[2], 0x06020400u);
    const u32 s_lo = __builtin_amdgcn_perm(p23, p01, 0x05040100u), s_hi = __builtin_amdgcn_perm(p23, p01, 0x07060302u);
    tag[u] = !valid || fit3 ? 0u : (fit4 ? 1u : 3u);
    g24[u] = valid ? (cacc & 0xFFFu) | ((cacc >> 16) << 12) : 0u;
    slo[u] = valid ? s_lo : 0u; shi[u] = valid ? s_hi : 0u;
    eb[u] = ((xacc >> 3) & 0xFu) | ((xacc >> 19) << 4);
  }
  // tag word of line a: this lane owns bits 8q..8q+7 (its four units)
  reinterpret_cast<uint8_t*>(L.tags)[4 * a + q] = (uint8_t)(tag[0] | (tag[1] << 2) | (tag[2] << 4) | (tag[3] << 6));
  u32x4 s0 = {slo[0], shi[0], slo[1], shi[1]}, s1 = {slo[2], shi[2], slo[3], shi[3]};
  *reinterpret_cast<u32x4*>(sm_tile + 16 * lane) = s0;
  *reinterpret_cast<u32x4*>(sm_tile + 1024 + 16 * lane) = s1;
  *reinterpret_cast<u32*>(cd_tile + 4 * lane) = g24[0] | (g24[1] << 24);
  *reinterpret_cast<u32*>(cd_tile + 256 + 4 * lane) = (g24[1] >> 8) | (g24[2] << 16);
  *reinterpret_cast<u32*>(cd_tile + 512 + 4 * lane) = (g24[2] >> 16) | (g24[3] << 8);
  wave_lds_sync();
  {
    const u32 f = L.tags[a];
    const u32 rb = (u32)esc_bytes(f), incl = row_scan16(rb);
    if (lane < T) { L.rowoff[lane] = (int)(incl - rb); flags_tile[lane] = (int)f; if (lane == T - 1) L.rowoff[T] = (int)incl; }
  }
  wave_lds_sync();
  if (esc_dst) {
    uint8_t* p = esc_dst + L.rowoff[a] + esc_prefix(L.tags[a], 8 * q);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (tag[u] == 1u) { p[0] = (uint8_t)eb[u]; p += 1; }
      else if (tag[u] == 3u) {
        // raw group: the upper five exponent bits of the eight elements, 40 bits little-endian (element i at bit 5i)
        u32 hl = 0u, hh = 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) { hl |= ((ew[u][i] >> 3) & 0x1Fu) << (5 * i); hh |= ((ew[u][i] >> 19) & 0x1Fu) << (5 * i); }
        const u64 h = (u64)hl | ((u64)hh << 20);
#pragma unroll
        for (int k = 0; k < 5; ++k) p[k] = (uint8_t)(h >> (8 * k));
        p += 5;
      }
    }
  }
  return L.rowoff[T];
}

// Per-lane metadata of a stored tile: the 2-bit tag of each of the lane's four units and the offset of the unit's escape
// bytes from the start of the tile's escape bytes.  tag_word = the tag word of the lane's line, flags_tile[lane & 15].
struct UnitMeta { u32 tag[4]; int pos[4]; };
__device__ __forceinline__ void tile_unit_meta(u32 tag_word, int lane, UnitMeta& M) {
  const int q = lane >> 4;
  const u32 rb = (u32)esc_bytes(tag_word);
  int pos = (int)(row_scan16(rb) - rb) + esc_prefix(tag_word, 8 * q);
#pragma unroll
  for (int u = 0; u < 4; ++u) { M.tag[u] = (tag_word >> (8 * q + 2 * u)) & 3u; M.pos[u] = pos; pos += tag_size(M.tag[u]); }
}

// Decodes one stored tile (native order) into 16 rows of 128 BF16 in natural channel order: row `tok` at out + tok*row_stride,
// rows >= nvalid are not written.  esc: the tile's escape bytes; b3row / b4row: the 128 base bytes of the head (channel order).
// One wave; bit-exact inverse of encode_staged_tile (codec.py:186-218).
template <int KIND>
__device__ __forceinline__ void decode_tile_rows(const uint8_t* __restrict__ sm_tile, const uint8_t* __restrict__ cd_tile,
                                                 const int* __restrict__ flags_tile, const uint8_t* __restrict__ esc,
                                                 const uint8_t* __restrict__ b3row, const uint8_t* __restrict__ b4row, int lane, int nvalid,
                                                 u16* __restrict__ out, long row_stride) {
  const int a = lane & 15, q = lane >> 4;
  Payload P;
  load_payload(sm_tile, cd_tile, lane, P);
  UnitMeta M;
  tile_unit_meta((u32)flags_tile[a], lane, M);
  u32 b3w[4], b4w[4];
  if (KIND == KIND_V) { load_base_words<KIND>(b3row, a, b3w); load_base_words<KIND>(b4row, a, b4w); }
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int tok = unit_token<KIND>(a, q, u), grp = unit_group<KIND>(a, q, u);
    if (KIND == KIND_K) { load_base_words<KIND>(b3row, grp, b3w); load_base_words<KIND>(b4row, grp, b4w); }
    u32 slo, shi, w[4];
    unit_sm(P, u, slo, shi);
    const u32 eb = M.tag[u] == 1u ? (u32)esc[M.pos[u]] : 0u;
    decode_unit(slo, shi, unit_code_word(P.c0, P.c1, P.c2, u), M.tag[u], eb, esc + M.pos[u], b3w, b4w, w);
    if (tok < nvalid) {
      u16* o = out + (long)tok * row_stride;
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        o[chan_of<KIND>(8 * grp + p)] = (u16)(w[p] & 0xFFFFu);
        o[chan_of<KIND>(8 * grp + p + 4)] = (u16)(w[p] >> 16);
      }
    }
  }
}

// decode_tile_rows through an LDS staging tile (T rows of STAGE_ROW u16, owned by the calling wave): the channel permutation turns the
// decoder's output into 2-byte scattered stores, which LDS absorbs; global memory then gets 16-byte stores, a full 256-byte row per
// 16 lanes.  Rows are padded by 16 bytes: the sixteen lanes of a K line write sixteen different rows at the same column, which an
// unpadded row stride (64 banks' worth) would send to one bank.
constexpr int STAGE_ROW = D + 8;
template <int KIND>
__device__ __forceinline__ void decode_tile_staged(const uint8_t* __restrict__ sm_tile, const uint8_t* __restrict__ cd_tile,
                                                   const int* __restrict__ flags_tile, const uint8_t* __restrict__ esc,
                                                   const uint8_t* __restrict__ b3row, const uint8_t* __restrict__ b4row, int lane, int nvalid,
                                                   u16* __restrict__ stage, u16* __restrict__ out, long row_stride) {
  decode_tile_rows<KIND>(sm_tile, cd_tile, flags_tile, esc, b3row, b4row, lane, T, stage, STAGE_ROW);
  wave_lds_sync();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    if (row < nvalid) *reinterpret_cast<u32x4*>(out + (long)row * row_stride + c16 * 8) = *reinterpret_cast<const u32x4*>(stage + row * STAGE_ROW + c16 * 8);
  }
}

}  // namespace gaac
