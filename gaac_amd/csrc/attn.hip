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

struct TileRegs {                // one lane's view of a (K tile, V tile) pair
  Payload k, v;
  UnitMeta km, vm;
  u32 keb[4], veb[4];
  const uint8_t* kesc; const uint8_t* vesc;
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

// ---------------------------------------------------------------------------------------------------- tile loaders
__device__ __forceinline__ void load_tags(const AttnArgs& A, long rowb, long tileb, int tile, int S, int a, u32& kfl, u32& vfl,
                                          int& ktoff, int& vtoff) {
  const int tok = tile * T + a;
  kfl = tok < S ? (u32)A.k.flags[rowb + tok] : 0u;
  vfl = tok < S ? (u32)A.v.flags[rowb + tok] : 0u;
  ktoff = A.k.tile_off[tileb + tile];
  vtoff = A.v.tile_off[tileb + tile];
}
__device__ __forceinline__ void load_tile(const AttnArgs& A, long rowb, int tile, int lane, u32 kfl, u32 vfl,
                                          const uint8_t* kesc, const uint8_t* vesc, TileRegs& R) {
  const long row0 = rowb + (long)tile * T;
  load_payload(A.k.sm + row0 * D, A.k.cd + row0 * CB, lane, R.k);
  load_payload(A.v.sm + row0 * D, A.v.cd + row0 * CB, lane, R.v);
  tile_unit_meta<KIND_K>(kfl, lane, R.km);
  tile_unit_meta<KIND_V>(vfl, lane, R.vm);
  R.kesc = kesc; R.vesc = vesc;
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    R.keb[u] = R.km.tag[u] == 1u ? (u32)kesc[R.km.pos[u]] : 0u;
    R.veb[u] = R.vm.tag[u] == 1u ? (u32)vesc[R.vm.pos[u]] : 0u;
  }
}

// ---------------------------------------------------------------------------------------------------- one tile pair
struct WaveState { f32x4 acc[8]; float m_run, l_run; };     // acc[i][r] = O[head a][group 4q+r, element i]

__device__ __forceinline__ void consume_tile(const TileRegs& R, WaveState& st, int tile, int S, float scale_log2e, int a, int q,
                                             const u32x4 (&qf)[4], const u32 (&kb3)[4][4], const u32 (&kb4)[4][4],
                                             const u32 (&vb3)[4], const u32 (&vb4)[4]) {
  // ---- scores: S[tok 4q+r][head a]
  f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi, w[4];
    unit_sm(R.k, u, slo, shi);
    decode_unit(slo, shi, unit_code_word(R.k.c0, R.k.c1, R.k.c2, u), R.km.tag[u], R.keb[u], R.kesc + R.km.pos[u], kb3[u], kb4[u], w);
    const u32x4 av = {w[0], w[1], w[2], w[3]};
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, qf[u]), sacc, 0, 0, 0);
  }
  // ---- online softmax per head a over the tile's 16 tokens (4 in this lane, 4 quads)
  const int tok0 = tile * T + 4 * q;
  float s[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) s[r] = tok0 + r < S ? sacc[r] * scale_log2e : -INFINITY;
  const float tmax = quad_rows_max(fmaxf(fmaxf(s[0], s[1]), fmaxf(s[2], s[3])));
  const float mn = fmaxf(st.m_run, tmax), mu = mn == -INFINITY ? 0.f : mn;
  const float alpha = __builtin_amdgcn_exp2f(st.m_run - mu);
  float p[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(s[r] - mu);
  st.l_run = st.l_run * alpha + ((p[0] + p[1]) + (p[2] + p[3]));
  st.m_run = mn;
  if (__builtin_amdgcn_ballot_w64(alpha != 1.f)) {
#pragma unroll
    for (int i = 0; i < 8; ++i) st.acc[i] *= alpha;
  }
  const u32x2 pw = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3])};
  const s16x4 pb = __builtin_bit_cast(s16x4, pw);
  // ---- values: decode the lane's 4 tokens of group a, regroup as token pairs per element, accumulate O^T
  u32 W[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi;
    unit_sm(R.v, u, slo, shi);
    decode_unit(slo, shi, unit_code_word(R.v.c0, R.v.c1, R.v.c2, u), R.vm.tag[u], R.veb[u], R.vesc + R.vm.pos[u], vb3, vb4, W[u]);
  }
  if (tile * T + T > S) {       // last, partly filled tile: rows beyond the sequence must not reach the product
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
  const int bh = blockIdx.x, split = blockIdx.y, tid = threadIdx.x;
  const int b = bh / A.n_kv, kvh = bh % A.n_kv, G = A.G;
  const int slot = A.slot[b], ch = (slot < 0 ? 0 : slot) * A.n_kv + kvh;
  if (split == A.nsplit) { tail_block(A, b, kvh, ch, slot); return; }

  const int S = slot < 0 ? 0 : A.sl[ch];
  const int ntiles = (S + T - 1) / T, chunk = (ntiles + A.nsplit - 1) / A.nsplit;
  const int tlo = split * chunk, thi = min(tlo + chunk, ntiles);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, a = lane & 15, q = lane >> 4;
  const long rowb = (long)ch * A.S_pad, tileb = (long)ch * (A.S_pad / T);
  const long qh0 = (long)b * A.n_q + (long)kvh * G;
  const uint8_t* ovk = A.k.ovf + A.k.head_start[ch];
  const uint8_t* ovv = A.v.ovf + A.v.head_start[ch];

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

  WaveState st;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m_run = -INFINITY; st.l_run = 0.f;

  TileRegs R0, R1;                 // ping-pong: one is consumed while the other is being loaded
  u32 kflN = 0u, vflN = 0u; int ktoN = 0, vtoN = 0;
  int tile = tlo + wave;
  if (tile < thi) {
    u32 kf, vf; int kto, vto;
    load_tags(A, rowb, tileb, tile, S, a, kf, vf, kto, vto);
    if (tile + 4 < thi) load_tags(A, rowb, tileb, tile + 4, S, a, kflN, vflN, ktoN, vtoN);
    load_tile(A, rowb, tile, lane, kf, vf, ovk + kto, ovv + vto, R0);
  }
  for (; tile < thi; tile += 8) {
    if (tile + 4 < thi) {
      load_tile(A, rowb, tile + 4, lane, kflN, vflN, ovk + ktoN, ovv + vtoN, R1);
      if (tile + 8 < thi) load_tags(A, rowb, tileb, tile + 8, S, a, kflN, vflN, ktoN, vtoN);
    }
    consume_tile(R0, st, tile, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
    if (tile + 4 >= thi) break;
    if (tile + 8 < thi) {
      load_tile(A, rowb, tile + 8, lane, kflN, vflN, ovk + ktoN, ovv + vtoN, R0);
      if (tile + 12 < thi) load_tags(A, rowb, tileb, tile + 12, S, a, kflN, vflN, ktoN, vtoN);
    }
    consume_tile(R1, st, tile + 4, S, A.scale_log2e, a, q, qf, kb3, kb4, vb3, vb4);
  }
  float m_run = st.m_run, l_run = st.l_run;
  f32x4 (&acc)[8] = st.acc;

  // ---- merge the 4 waves of the block, write the split's partial
  __shared__ float sh_m[4][GMAX], sh_l[4][GMAX];
  __shared__ float sh_acc[4][GMAX][D];
  l_run = quad_rows_sum(l_run);
  if (a < G) {
    if (q == 0) { sh_m[wave][a] = m_run; sh_l[wave][a] = l_run; }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) sh_acc[wave][a][chan_v(8 * (4 * q + r) + i)] = acc[i][r];
  }
  __syncthreads();
  const int d = tid & 127;
  for (int g = tid >> 7; g < G; g += 2) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, sh_m[w][g]);
    float Lc = 0.f, Ac = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = sh_m[w][g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(sh_m[w][g] - M);
      Lc += sh_l[w][g] * f; Ac += sh_acc[w][g][d] * f;
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
