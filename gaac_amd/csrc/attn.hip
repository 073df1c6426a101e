// Fused split-K decode attention over compressed K/V for gfx950 (wave64, MFMA), the raw-BF16 tail, and the split merge.
// Counterpart of gaac_attn / gaac_tail / gaac_combine / gaac_attn_launch in /root/reference/gaac/kernel.py:48-326
// (same inputs, same partial (m, l, acc) protocol, same slot map and padded-row behaviour), redesigned for CDNA4:
//
//   * one block = (batch row, kv head, split), 4 waves; wave w streams tiles tlo+w, tlo+w+4, ... of the split;
//   * scores   S[16 tok x 16 heads]  = K[16 x 128] . Q^T      : 4 x v_mfma_f32_16x16x32_bf16   (A = decoded K units)
//   * output   O^T[128 x 16 heads]  += V^T[128 x 16] . P^T     : 8 x v_mfma_f32_16x16x16_bf16   (A = decoded V units)
//     The score tile lands in the register layout the second product wants for P^T, so P never crosses lanes.
//   * the GQA group (<= 16 query heads) rides in the N dimension; register use does not depend on it;
//   * three-stage prefetch per wave: tag words of tile t+8, payload + escape bytes of tile t+4, consume tile t;
//   * the tail (<= 16 raw BF16 tokens per head) is one extra block row of the same launch; its partial goes to the
//     last partial slot.  Softmax runs in base 2 (scale * log2 e folded into the scores).
#include "gaac_tile.h"
#include "gaac_capi.h"
#include "../../include/gaac_hip.h"

namespace gaac {

constexpr int GMAX = 16;         // query heads per kv head the MFMA tile can carry
constexpr int MAX_SLOTS = 1024;  // split partials a combine block can merge

struct StoreView {               // one kind (K or V) of a page or of a cache store
  const uint8_t* sm; const uint8_t* cd; const int* flags; const int* tile_off; const uint8_t* ovf; const int* head_start;
  const uint8_t* base3; const uint8_t* base4;
};
struct AttnArgs {
  StoreView k, v;
  const u16* q; float* pm; float* pl; float* pa;
  const int* slot; const int* sl;
  int S_pad; float scale_log2e; int nsplit; int nslot; int n_kv; int n_q; int G; int NB;
  const u16* kt; const u16* vt; const int* tl; int tcap;
};

__device__ __forceinline__ float bf16_bits_to_float(u32 h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ u32 pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 v; v[0] = (__bf16)lo; v[1] = (__bf16)hi;
  return __builtin_bit_cast(u32, v);
}

// ---------------------------------------------------------------------------------------------------- raw tail block
__device__ void tail_block(const AttnArgs& A, int b, int kvh, int ch, int slot) {
  __shared__ float qs[GMAX][D];
  __shared__ float sc[GMAX][T];
  const int tid = threadIdx.x, G = A.G;
  const int TL = slot < 0 ? 0 : min(A.tl[ch], A.tcap);
  const long qh0 = (long)b * A.n_q + (long)kvh * G;
  for (int i = tid; i < G * D; i += 256) qs[i >> 7][i & 127] = bf16_bits_to_float(A.q[qh0 * D + i]);
  __syncthreads();
  const int t = tid >> 4, c = tid & 15;
  const long base = (long)ch * A.tcap * D;
  float kr[8];
  {
    u32x4 kv = {0u, 0u, 0u, 0u};
    if (t < TL) kv = *reinterpret_cast<const u32x4*>(A.kt + base + (long)t * D + 8 * c);
#pragma unroll
    for (int i = 0; i < 4; ++i) { kr[2 * i] = bf16_bits_to_float(kv[i] & 0xFFFFu); kr[2 * i + 1] = bf16_bits_to_float(kv[i] >> 16); }
  }
  for (int g = 0; g < G; ++g) {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d += qs[g][8 * c + i] * kr[i];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) d += __shfl_xor(d, o, 16);
    if (c == 0) sc[g][t] = t < TL ? d * A.scale_log2e : -INFINITY;
  }
  __syncthreads();
  {   // thread (g = tid >> 4, token = tid & 15): softmax over the 16 lanes of the row
    const int g = tid >> 4, tk = tid & 15;
    float s = g < G ? sc[g][tk] : -INFINITY, m = s;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 16));
    const float mu = m == -INFINITY ? 0.f : m;
    const float p = __builtin_amdgcn_exp2f(s - mu);
    float l = p;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) l += __shfl_xor(l, o, 16);
    __syncthreads();
    if (g < G) {
      sc[g][tk] = p;
      if (tk == 0) { const long pidx = (qh0 + g) * A.nslot + (A.nslot - 1); A.pm[pidx] = m; A.pl[pidx] = l; }
    }
  }
  __syncthreads();
  const int d = tid & 127;
  for (int g = tid >> 7; g < G; g += 2) {
    float acc = 0.f;
    for (int tk = 0; tk < TL; ++tk) acc += sc[g][tk] * bf16_bits_to_float(A.vt[base + (long)tk * D + d]);
    A.pa[((qh0 + g) * A.nslot + (A.nslot - 1)) * D + d] = acc;
  }
}

// ---------------------------------------------------------------------------------------------------- lookup tables
// xlut[e]: the four exponent-field words carrying the 4th code bits of escape byte e (bit p -> element p, bit 4+p -> element p+4).
// sel[m]:  v_perm selector that spreads a lane's packed 4-bit-group escape bytes to one byte per unit; m has bit 2u set when
//          unit u owns an escape byte; byte u of the selector = index of that byte among the lane's bytes, or 0x0C (-> 0).
struct AttnLds {
  u32x4 xlut[256];
  u32 sel[96];
  float m[4][GMAX], l[4][GMAX];
  float acc[4][GMAX][D];
};
__device__ __forceinline__ void build_luts(AttnLds& L, int tid) {
  {
    const u32 e = (u32)tid;
    u32x4 w;
#pragma unroll
    for (int p = 0; p < 4; ++p) w[p] = (((e >> p) & 1u) << 10) | (((e >> (4 + p)) & 1u) << 26);
    L.xlut[tid] = w;
  }
  if (tid < 96) {
    u32 selw = 0u, n = 0u;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const bool has = (tid >> (2 * u)) & 1;
      selw |= (has ? n : 0x0Cu) << (8 * u);
      n += has ? 1u : 0u;
    }
    L.sel[tid] = selw;
  }
}

// ---------------------------------------------------------------------------------------------------- tile loaders
struct TileRegs {                // one lane's view of a (K tile, V tile) pair
  Payload k, v;
  u32 kf;                        // tag word of token a (K)
  u32 kpos0;                     // offset of the lane's first K unit in the tile's escape bytes
  u32x2 ke;                      // 8 escape bytes from kpos0 on
  u32 vt8;                       // tags of the lane's 4 V units, 2 bits each
  u32 vpos[4];                   // offsets of the 4 V units in the tile's escape bytes
  u32x2 ve[4];                   // 8 escape bytes from each V unit's offset on
};
struct TagRegs { u32 kfl, vfl; u32 kto, vto; };

struct Bases {                   // uniform (scalar) views of one cache head
  const uint8_t* ksm; const uint8_t* kcd; const int* kfl; const int* kto; const uint8_t* kov;
  const uint8_t* vsm; const uint8_t* vcd; const int* vfl; const int* vto; const uint8_t* vov;
};

__device__ __forceinline__ void load_tags(const Bases& B, int tile, int S, int a, TagRegs& Tg) {
  const unsigned tok = (unsigned)(tile * T + a);
  Tg.kfl = (u32)B.kfl[tok]; Tg.vfl = (u32)B.vfl[tok];
  if ((int)tok >= S) { Tg.kfl = 0u; Tg.vfl = 0u; }
  Tg.kto = (u32)B.kto[tile]; Tg.vto = (u32)B.vto[tile];
}

__device__ __forceinline__ void load_tile(const Bases& B, int tile, int lane, const TagRegs& Tg, const u32 (&bperm_addr)[4], TileRegs& R) {
  const int a = lane & 15, q = lane >> 4;
  load_payload(B.ksm + (size_t)tile * TILE_SM, B.kcd + (size_t)tile * TILE_CD, lane, R.k);
  load_payload(B.vsm + (size_t)tile * TILE_SM, B.vcd + (size_t)tile * TILE_CD, lane, R.v);
  // per-row escape bytes of K (low half) and V (high half), one scan for both
  const u32 rb = (u32)esc_bytes(Tg.kfl) | ((u32)esc_bytes(Tg.vfl) << 16);
  const u32 excl = row_scan16(rb) - rb;
  R.kf = Tg.kfl;
  R.kpos0 = (excl & 0xFFFFu) + (u32)esc_prefix(Tg.kfl, 8 * q);
  R.ke = load_u32x2_unaligned(B.kov + Tg.kto + R.kpos0);
  const u32 rov = excl >> 16;
  R.vt8 = 0u;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const u32 f = (u32)__builtin_amdgcn_ds_bpermute((int)bperm_addr[u], (int)Tg.vfl);
    const u32 ro = (u32)__builtin_amdgcn_ds_bpermute((int)bperm_addr[u], (int)rov);
    R.vt8 |= ((f >> (2 * a)) & 3u) << (2 * u);
    R.vpos[u] = ro + (u32)esc_prefix(f, 2 * a);
    R.ve[u] = load_u32x2_unaligned(B.vov + Tg.vto + R.vpos[u]);
  }
}

// ---------------------------------------------------------------------------------------------------- one tile pair
struct WaveState { f32x4 acc[8]; float m_run, mu_run, l_run; };     // acc[i][r] = O[head a][group 4q+r, element i]

// unit decode with the escape contribution already expanded to exponent-field words x (see AttnLds::xlut)
__device__ __forceinline__ void decode_unit_x(u32 slo, u32 shi, u32 g24, bool t0, const u32x4& x, const u32* __restrict__ b3w,
                                              const u32* __restrict__ b4w, u32* __restrict__ out) {
  const u32 cw = (g24 & 0xFFFu) | ((g24 << 4) & 0x0FFF0000u);
  const u32 c0 = (cw << 7) & 0x03800380u, c1 = (cw << 4) & 0x03800380u, c2 = (cw << 1) & 0x03800380u, c3 = (cw >> 2) & 0x03800380u;
  const u32 e0 = c0 + (t0 ? b3w[0] : b4w[0]) + x[0], e1 = c1 + (t0 ? b3w[1] : b4w[1]) + x[1];
  const u32 e2 = c2 + (t0 ? b3w[2] : b4w[2]) + x[2], e3 = c3 + (t0 ? b3w[3] : b4w[3]) + x[3];
  out[0] = (e0 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x04040000u) & ~EXP_MASK2);
  out[1] = (e1 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x05050101u) & ~EXP_MASK2);
  out[2] = (e2 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x06060202u) & ~EXP_MASK2);
  out[3] = (e3 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x07070303u) & ~EXP_MASK2);
}
// raw group: 8 x 5 high exponent bits (40-bit little endian in lo/hi) as exponent-field words MINUS the 4-bit base words,
// so that code + base4 + x reproduces code | hi5 << 3 exactly (32-bit arithmetic, the base cancels)
__device__ __forceinline__ u32x4 raw_x_words(u32 lo, u32 hi, const u32* __restrict__ b4w) {
  u32x4 x;
  x[0] = (((lo) & 31u) << 10 | ((lo >> 20) & 31u) << 26) - b4w[0];
  x[1] = (((lo >> 5) & 31u) << 10 | ((lo >> 25) & 31u) << 26) - b4w[1];
  x[2] = (((lo >> 10) & 31u) << 10 | (__builtin_amdgcn_alignbit(hi, lo, 30) & 31u) << 26) - b4w[2];
  x[3] = (((lo >> 15) & 31u) << 10 | ((hi >> 3) & 31u) << 26) - b4w[3];
  return x;
}

__device__ __forceinline__ void consume_tile(const TileRegs& R, WaveState& st, AttnLds& L, const Bases& B,
                                             u32 kto, u32 vto, int tile, int S, float scale_log2e, int a, int q,
                                             const u32x4 (&qf)[4], const u32 (&kb3)[4][4], const u32 (&kb4)[4][4],
                                             const u32 (&vb3)[4], const u32 (&vb4)[4]) {
  // ---- K escapes: spread the lane's 4-bit-group bytes to units, expand through the table
  const u32 ktag8 = __builtin_amdgcn_ubfe(R.kf, 8 * q, 8);
  u32x4 x[4];
  {
    const u32 eb4 = __builtin_amdgcn_perm(0u, R.ke[0], L.sel[ktag8 & 0x55u]);
#pragma unroll
    for (int u = 0; u < 4; ++u) x[u] = L.xlut[(eb4 >> (8 * u)) & 0xFFu];
  }
  if (__builtin_amdgcn_ballot_w64((ktag8 & 0xAAu) != 0u)) {      // some lane holds a raw group (rare per lane, common per tile)
    if (ktag8 & 0xAAu) {                                          // redo every escaped unit of this lane at its true offset
      u32 off = 0u;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const u32 t = (ktag8 >> (2 * u)) & 3u;
        if (t) {
          u32 lo, hi;
          if (off + (u32)tag_size(t) <= 8u) {
            const u64 v = ((u64)R.ke[0] | ((u64)R.ke[1] << 32)) >> (8u * off);
            lo = (u32)v; hi = (u32)(v >> 32);
          } else {
            const u64 v = load_u64_unaligned(B.kov + kto + R.kpos0 + off);
            lo = (u32)v; hi = (u32)(v >> 32);
          }
          x[u] = t == 1u ? L.xlut[lo & 0xFFu] : raw_x_words(lo, hi, kb4[u]);
        }
        off += (u32)tag_size(t);
      }
    }
  }
  // ---- scores: S[tok 4q+r][head a]
  f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi, w[4];
    unit_sm(R.k, u, slo, shi);
    decode_unit_x(slo, shi, unit_code_word(R.k.c0, R.k.c1, R.k.c2, u), ((ktag8 >> (2 * u)) & 1u) == 0u, x[u], kb3[u], kb4[u], w);
    const u32x4 av = {w[0], w[1], w[2], w[3]};
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, qf[u]), sacc, 0, 0, 0);
  }
  // ---- V escapes (each unit has its own 8 bytes)
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const bool t0 = ((R.vt8 >> (2 * u)) & 1u) == 0u;
    x[u] = L.xlut[t0 ? 0u : (R.ve[u][0] & 0xFFu)];
  }
  if (__builtin_amdgcn_ballot_w64((R.vt8 & 0xAAu) != 0u)) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (((R.vt8 >> (2 * u)) & 3u) == 3u) x[u] = raw_x_words(R.ve[u][0], R.ve[u][1], vb4);
  }
  // ---- online softmax per head a over the tile's 16 tokens (4 in this lane, 4 quads), base 2
  const int tok0 = tile * T + 4 * q;
  float s[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = sacc[r] * scale_log2e;
  const bool partial = tile * T + T > S;          // uniform: only the last tile of a sequence can be partly filled
  if (partial) {
#pragma unroll
    for (int r = 0; r < 4; ++r) if (tok0 + r >= S) s[r] = -INFINITY;
  }
  const float tmax = quad_rows_max(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
  if (__builtin_amdgcn_ballot_w64(tmax > st.m_run)) {             // the running maximum of some head grows (rare after the first tiles)
    const float mn = fmaxf(st.m_run, tmax), mu = mn == -INFINITY ? 0.f : mn;
    const float alpha = __builtin_amdgcn_exp2f(st.m_run - mu);
    st.l_run *= alpha;
#pragma unroll
    for (int i = 0; i < 8; ++i) st.acc[i] *= alpha;
    st.m_run = mn; st.mu_run = mu;
  }
  float p[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(s[r] - st.mu_run);
  st.l_run += (p[0] + p[1]) + (p[2] + p[3]);
  const u32x2 pw = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3])};
  const s16x4 pb = __builtin_bit_cast(s16x4, pw);
  // ---- values: decode the lane's 4 tokens of group a, regroup as token pairs per element, accumulate O^T
  u32 W[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi;
    unit_sm(R.v, u, slo, shi);
    decode_unit_x(slo, shi, unit_code_word(R.v.c0, R.v.c1, R.v.c2, u), ((R.vt8 >> (2 * u)) & 1u) == 0u, x[u], vb3, vb4, W[u]);
  }
  if (partial) {                // rows beyond the sequence must not reach the product
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (tok0 + u >= S) { W[u][0] = W[u][1] = W[u][2] = W[u][3] = 0u; }
  }
#pragma unroll
  for (int pp = 0; pp < 4; ++pp) {
    const u32x2 lo = {__builtin_amdgcn_perm(W[1][pp], W[0][pp], 0x05040100u), __builtin_amdgcn_perm(W[3][pp], W[2][pp], 0x05040100u)};
    const u32x2 hi = {__builtin_amdgcn_perm(W[1][pp], W[0][pp], 0x07060302u), __builtin_amdgcn_perm(W[3][pp], W[2][pp], 0x07060302u)};
    st.acc[pp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, lo), pb, st.acc[pp], 0, 0, 0);
    st.acc[pp + 4] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, hi), pb, st.acc[pp + 4], 0, 0, 0);
  }
}

// ---------------------------------------------------------------------------------------------------- main kernel
__global__ void __launch_bounds__(256, 2) k_attn_split(const AttnArgs A) {
  __shared__ AttnLds L;
  const int bh = blockIdx.x, split = blockIdx.y, tid = threadIdx.x;
  const int b = bh / A.n_kv, kvh = bh % A.n_kv, G = A.G;
  const int slot = A.slot[b], ch = (slot < 0 ? 0 : slot) * A.n_kv + kvh;
  if (split == A.nsplit) { tail_block(A, b, kvh, ch, slot); return; }
  build_luts(L, tid);

  const int S = slot < 0 ? 0 : A.sl[ch];
  const int ntiles = (S + T - 1) / T, chunk = (ntiles + A.nsplit - 1) / A.nsplit;
  const int tlo = split * chunk, thi = min(tlo + chunk, ntiles);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, a = lane & 15, q = lane >> 4;
  const long rowb = (long)ch * A.S_pad, tileb = (long)ch * (A.S_pad / T);
  const long qh0 = (long)b * A.n_q + (long)kvh * G;
  Bases B;
  B.ksm = A.k.sm + rowb * D; B.kcd = A.k.cd + rowb * CB; B.kfl = A.k.flags + rowb; B.kto = A.k.tile_off + tileb; B.kov = A.k.ovf + A.k.head_start[ch];
  B.vsm = A.v.sm + rowb * D; B.vcd = A.v.cd + rowb * CB; B.vfl = A.v.flags + rowb; B.vto = A.v.tile_off + tileb; B.vov = A.v.ovf + A.v.head_start[ch];

  // Q as the B operand of the score product: lane (head a, quad q), product u covers group 4q+u in word order (e, e+4)
  u32x4 qf[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      u32 w = 0u;
      if (a < G) {
        const u16* qp = A.q + (qh0 + a) * D;
        w = (u32)qp[chan_k(8 * (4 * q + u) + p)] | ((u32)qp[chan_k(8 * (4 * q + u) + p + 4)] << 16);
      }
      qf[u][p] = w;
    }
  }
  // exponent-base words of the lane's units
  const int brow = ch % A.NB;
  u32 kb3[4][4], kb4[4][4], vb3[4], vb4[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    load_base_words<KIND_K>(A.k.base3 + (long)brow * D, 4 * q + u, kb3[u]);
    load_base_words<KIND_K>(A.k.base4 + (long)brow * D, 4 * q + u, kb4[u]);
  }
  load_base_words<KIND_V>(A.v.base3 + (long)brow * D, a, vb3);
  load_base_words<KIND_V>(A.v.base4 + (long)brow * D, a, vb4);
  u32 bperm_addr[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) bperm_addr[u] = (u32)(4 * (4 * q + u));
  __syncthreads();        // lookup tables are ready

  WaveState st;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m_run = -INFINITY; st.mu_run = 0.f; st.l_run = 0.f;

  // tiles of this wave: t(i) = tlo + wave + 4 i, i < n.  Ping-pong registers R0/R1; tag words are fetched one tile further
  // ahead (index clamped to the wave's last tile, so that no load sits under a branch the consumer has to join).
  const int t0 = tlo + wave;
  const int n = t0 < thi ? (thi - t0 + 3) / 4 : 0;
  if (n > 0) {
    const int tlast = t0 + 4 * (n - 1);
    TileRegs R0, R1;
    TagRegs Tg, TgC0, TgC1;
    load_tags(B, t0, S, a, Tg);
    TgC0 = Tg;
    load_tile(B, t0, lane, Tg, bperm_addr, R0);
    load_tags(B, min(t0 + 4, tlast), S, a, Tg);
    int i = 0;
    for (; i + 2 < n; i += 2) {
      const int t = t0 + 4 * i;
      TgC1 = Tg;
      load_tile(B, t + 4, lane, Tg, bperm_addr, R1);
      load_tags(B, min(t + 8, tlast), S, a, Tg);
      consume_tile(R0, st, L, B, TgC0.kto, TgC0.vto, t, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
      TgC0 = Tg;
      load_tile(B, t + 8, lane, Tg, bperm_addr, R0);
      load_tags(B, min(t + 12, tlast), S, a, Tg);
      consume_tile(R1, st, L, B, TgC1.kto, TgC1.vto, t + 4, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
    }
    const int t = t0 + 4 * i;
    if (n - i == 2) {
      TgC1 = Tg;
      load_tile(B, t + 4, lane, Tg, bperm_addr, R1);
      consume_tile(R0, st, L, B, TgC0.kto, TgC0.vto, t, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
      consume_tile(R1, st, L, B, TgC1.kto, TgC1.vto, t + 4, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
    } else {
      consume_tile(R0, st, L, B, TgC0.kto, TgC0.vto, t, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
    }
  }
  float m_run = st.m_run, l_run = st.l_run;
  f32x4 (&acc)[8] = st.acc;

  // ---- merge the 4 waves of the block, write the split's partial
  l_run = quad_rows_sum(l_run);
  if (a < G) {
    if (q == 0) { L.m[wave][a] = m_run; L.l[wave][a] = l_run; }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) L.acc[wave][a][chan_v(8 * (4 * q + r) + i)] = acc[i][r];
  }
  __syncthreads();
  const int d = tid & 127;
  for (int g = tid >> 7; g < G; g += 2) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, L.m[w][g]);
    float Lc = 0.f, Ac = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = L.m[w][g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(L.m[w][g] - M);
      Lc += L.l[w][g] * f; Ac += L.acc[w][g][d] * f;
    }
    const long pidx = (qh0 + g) * A.nslot + split;
    if (d == 0) { A.pm[pidx] = M; A.pl[pidx] = Lc; }
    A.pa[pidx * D + d] = Ac;
  }
}

// ---------------------------------------------------------------------------------------------------- split merge
__global__ void __launch_bounds__(128) k_attn_combine(const float* __restrict__ pm, const float* __restrict__ pl, const float* __restrict__ pa,
                                                      u16* __restrict__ out, int nslot) {
  __shared__ float fs[MAX_SLOTS];
  __shared__ float red[2];
  const int qh = blockIdx.x, tid = threadIdx.x;
  float m = -INFINITY;
  for (int s = tid; s < nslot; s += 128) m = fmaxf(m, pm[(long)qh * nslot + s]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63) == 0) red[tid >> 6] = m;
  __syncthreads();
  const float M = fmaxf(red[0], red[1]);
  __syncthreads();
  float l = 0.f;
  for (int s = tid; s < nslot; s += 128) {
    const float v = pm[(long)qh * nslot + s];
    const float f = v == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(v - M);
    fs[s] = f; l += pl[(long)qh * nslot + s] * f;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
  if ((tid & 63) == 0) red[tid >> 6] = l;
  __syncthreads();
  const float L = red[0] + red[1];
  float acc = 0.f;
  for (int s = 0; s < nslot; ++s) acc += pa[((long)qh * nslot + s) * D + tid] * fs[s];
  const float o = L > 0.f ? acc / L : 0.f;
  out[(long)qh * D + tid] = __builtin_bit_cast(u16, (__bf16)o);
}

}  // namespace gaac

using namespace gaac;

static int attn_split_impl(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, float* pm, float* pl, float* pa, void* stream) {
  GAAC_REQUIRE(n_kv > 0 && n_q > 0 && n_q % n_kv == 0 && n_q / n_kv >= 1 && n_q / n_kv <= GMAX, "GQA group size must be 1..%d (n_q=%d, n_kv=%d)", GMAX, n_q, n_kv);
  GAAC_REQUIRE(smk && ck && fk && tok && ovk && ohsk && b3k && b4k && smv && cv && fv && tov && ovv && ohsv && b3v && b4v, "gaac_attn: null store pointer");
  GAAC_REQUIRE(q && slot && SL && pm && pl && pa, "gaac_attn: null pointer");
  GAAC_REQUIRE(B > 0 && S_pad > 0 && S_pad % T == 0 && NB > 0, "gaac_attn: bad sizes B=%d S_pad=%d NB=%d", B, S_pad, NB);
  const bool has_tail = kt != nullptr;
  GAAC_REQUIRE(!has_tail || (vt && TL && TCAP >= 1 && TCAP <= T), "gaac_attn: tail needs kt, vt, TL and 1 <= TCAP <= %d", T);
  const int nslot = nsplit + (has_tail ? 1 : 0);
  GAAC_REQUIRE(nsplit >= 1 && nslot <= MAX_SLOTS, "gaac_attn: nsplit must be in 1..%d", MAX_SLOTS - 1);
  AttnArgs A;
  A.k = StoreView{smk, ck, fk, tok, ovk, ohsk, b3k, b4k};
  A.v = StoreView{smv, cv, fv, tov, ovv, ohsv, b3v, b4v};
  A.q = (const u16*)q; A.pm = pm; A.pl = pl; A.pa = pa; A.slot = slot; A.sl = SL;
  A.S_pad = S_pad; A.scale_log2e = scale * 1.4426950408889634f; A.nsplit = nsplit; A.nslot = nslot;
  A.n_kv = n_kv; A.n_q = n_q; A.G = n_q / n_kv; A.NB = NB;
  A.kt = (const u16*)kt; A.vt = (const u16*)vt; A.tl = TL; A.tcap = TCAP;
  hipLaunchKernelGGL(k_attn_split, dim3(B * n_kv, nslot), dim3(256), 0, (hipStream_t)stream, A);
  return launch_status("gaac_attn(split)");
}

extern "C" int gaac_attn_split(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, float* pm, float* pl, float* pa, void* stream) {
  return attn_split_impl(smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v, q, slot, B, n_q, n_kv, SL, S_pad,
                         scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, stream);
}

extern "C" int gaac_attn_combine(const float* pm, const float* pl, const float* pa, void* out, int n_rows, int nslot, void* stream) {
  GAAC_REQUIRE(pm && pl && pa && out && n_rows > 0 && nslot >= 1 && nslot <= MAX_SLOTS, "gaac_attn_combine: bad arguments");
  hipLaunchKernelGGL(k_attn_combine, dim3(n_rows), dim3(128), 0, (hipStream_t)stream, pm, pl, pa, (u16*)out, nslot);
  return launch_status("gaac_attn(combine)");
}

extern "C" int gaac_attn_launch(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP,
    float* pm, float* pl, float* pa, void* out, void* stream) {
  GAAC_REQUIRE(out, "gaac_attn_launch: null output");
  int rc = attn_split_impl(smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v, q, slot, B, n_q, n_kv, SL, S_pad,
                           scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, stream);
  if (rc) return rc;
  return gaac_attn_combine(pm, pl, pa, out, B * n_q, nsplit + (kt ? 1 : 0), stream);
}
