// Wave-level tile encoder and tile metadata helpers (one wave64 = one 16-token tile), shared by the page encoder,
// the cache append kernel and the paged store.  Tier rule, code words, tag words and escape bytes follow
// /root/reference/gaac/codec.py:138-172 and /root/reference/gaac/encoder.py:30-66; byte placement is the native one
// described in gaac_core.h.
#pragma once
#include "gaac_core.h"

namespace gaac {

// LDS scratch of one encoding wave
struct EncodeLds {
  u16 x[T * D];        // the tile's BF16 bit patterns, token-major, natural channel order (rows >= nvalid are zero)
  uint8_t b3[D], b4[D];
  u32 tags[T];
  int rowoff[T + 1];   // exclusive prefix of per-row escape bytes; [16] = tile total
};

// Stage 16 rows of 128 BF16 (row r at src + r*row_stride elements) into lds.x; rows >= nvalid read as zero.
__device__ __forceinline__ void stage_rows(EncodeLds& L, const u16* __restrict__ src, long row_stride, int nvalid, int lane) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (row < nvalid) v = *reinterpret_cast<const u32x4*>(src + (long)row * row_stride + c16 * 8);
    *reinterpret_cast<u32x4*>(&L.x[row * D + c16 * 8]) = v;
  }
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

// Encodes the tile staged in L (after a barrier).  Writes the native sign/mantissa and code bytes, the 16 tag words (one per line) and
// the escape bytes (at esc_dst + offset-in-tile; nullptr = count only).  Returns the tile's escape byte count (all lanes).
// Must be called by all 64 lanes of the wave that owns L; it synchronises that wave only.
template <int KIND>
__device__ __forceinline__ int encode_staged_tile(EncodeLds& L, int nvalid, int lane, uint8_t* __restrict__ sm_tile,
                                                  uint8_t* __restrict__ cd_tile, int* __restrict__ flags_tile,
                                                  uint8_t* __restrict__ esc_dst) {
  const int a = lane & 15, q = lane >> 4;
  u32 slo[4], shi[4], g24[4], tag[4], eb[4];
  u64 hi40[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const int tok = unit_token<KIND>(a, q, u), grp = unit_group<KIND>(a, q, u);
    bool fit3 = true, fit4 = true;
    u32 c3 = 0, c4 = 0, cr = 0, s_lo = 0, s_hi = 0, e4 = 0;
    u64 h = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int ch = chan_of<KIND>(8 * grp + i);
      const u32 x = L.x[tok * D + ch];
      const int e = (int)((x >> 7) & 0xFFu);
      const u32 smb = ((x >> 8) & 0x80u) | (x & 0x7Fu);
      const int d3 = e - (int)L.b3[ch], d4 = e - (int)L.b4[ch];
      fit3 = fit3 && ((unsigned)d3 < 8u);
      fit4 = fit4 && ((unsigned)d4 < 16u);
      c3 |= (u32)(d3 & 7) << (3 * i); c4 |= (u32)(d4 & 7) << (3 * i); cr |= (u32)(e & 7) << (3 * i);
      e4 |= (u32)((d4 >> 3) & 1) << i;
      h |= (u64)(e >> 3) << (5 * i);
      if (i < 4) s_lo |= smb << (8 * i); else s_hi |= smb << (8 * (i - 4));
    }
    const bool valid = tok < nvalid;          // padded rows: tier 0, code 0, sign/mantissa 0
    tag[u] = !valid || fit3 ? 0u : (fit4 ? 1u : 3u);
    g24[u] = !valid ? 0u : (fit3 ? c3 : (fit4 ? c4 : cr));
    slo[u] = valid ? s_lo : 0u; shi[u] = valid ? s_hi : 0u;
    eb[u] = e4; hi40[u] = h;
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
#pragma unroll
        for (int k = 0; k < 5; ++k) p[k] = (uint8_t)(hi40[u] >> (8 * k));
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

// decode_tile_rows through an LDS staging tile (T*D u16, owned by the calling wave): the channel permutation turns the decoder's
// output into 2-byte scattered stores, which LDS absorbs; global memory then gets 16-byte stores, a full 256-byte row per 16 lanes.
template <int KIND>
__device__ __forceinline__ void decode_tile_staged(const uint8_t* __restrict__ sm_tile, const uint8_t* __restrict__ cd_tile,
                                                   const int* __restrict__ flags_tile, const uint8_t* __restrict__ esc,
                                                   const uint8_t* __restrict__ b3row, const uint8_t* __restrict__ b4row, int lane, int nvalid,
                                                   u16* __restrict__ stage, u16* __restrict__ out, long row_stride) {
  decode_tile_rows<KIND>(sm_tile, cd_tile, flags_tile, esc, b3row, b4row, lane, T, stage, D);
  wave_lds_sync();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    if (row < nvalid) *reinterpret_cast<u32x4*>(out + (long)row * row_stride + c16 * 8) = *reinterpret_cast<const u32x4*>(stage + row * D + c16 * 8);
  }
}

}  // namespace gaac
