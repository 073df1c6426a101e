// Measurement aids of bench.py, built into libgaac_bench.so (not part of the product library libgaac_hip.so).
//
// gaac_stream_copy: a plain copy with 16-byte accesses per lane, the known-size kernel against which the HBM traffic counters
// (FETCH_SIZE / WRITE_SIZE) are scaled.
//
// gaac_read_probe / gaac_read_probe_paged: the memory side of the fused decode-attention kernel without its arithmetic.  One block per (cache head, split), eight
// waves, every wave fetches the tiles wave, wave + 8, ... of the block's contiguous range one tile ahead of the tile it "consumes" (an
// xor over the loaded registers), with the attention kernel's own loads: per tile and kind two 16-byte and three 4-byte loads per lane
// (non-temporal), and, on request, the tile's tag words, its offset in the escape stream and eight escape bytes per lane.  What this
// kernel needs for a page is what the load pattern itself costs on the part: the floor under k_attn_split for that page.
#include "gaac_tile.h"      // -I gaac_amd/csrc: the tile format and the payload loads of the attention kernel

namespace gaac {

struct ProbeView { const uint8_t* sm; const uint8_t* cd; const int* flags; const int* tile_off; const uint8_t* ovf; const int* head_start; };
struct ProbeRegs { Payload k, v; u32 kf, vf, kto, vto; u32x2 ke, ve; };

template <bool META>
__device__ __forceinline__ void probe_load(const ProbeView& K, const ProbeView& V, long rowb, long tileb, long khs, long vhs, int tile, int lane, ProbeRegs& R) {
  const u32 so = (u32)tile * TILE_SM, co = (u32)tile * TILE_CD;
  load_payload(K.sm + rowb * D + so, K.cd + rowb * CB + co, lane, R.k);
  load_payload(V.sm + rowb * D + so, V.cd + rowb * CB + co, lane, R.v);
  if (META) {
    const int a = lane & 15;
    R.kf = (u32)__builtin_nontemporal_load(K.flags + rowb + tile * T + a); R.vf = (u32)__builtin_nontemporal_load(V.flags + rowb + tile * T + a);
    R.kto = (u32)K.tile_off[tileb + tile]; R.vto = (u32)V.tile_off[tileb + tile];
  }
}
__device__ __forceinline__ u32 probe_fold(const ProbeRegs& R) {
  return R.k.s0[0] ^ R.k.s0[3] ^ R.k.s1[1] ^ R.k.s1[2] ^ R.k.c0 ^ R.k.c1 ^ R.k.c2 ^ R.v.s0[0] ^ R.v.s0[3] ^ R.v.s1[1] ^ R.v.s1[2] ^ R.v.c0 ^ R.v.c1 ^ R.v.c2;
}
// META: also the tag words, tile offsets and escape bytes (the escape loads wait for the tag words of their tile, as in the attention
// kernel: a lane's escape position is a prefix over the tag words)
template <bool META>
__global__ void __launch_bounds__(512, 1) k_read_probe(ProbeView K, ProbeView V, int S_pad, int ntiles, int nsplit, u32* __restrict__ sink) {
  constexpr int NW = 8;
  const int ch = (int)blockIdx.x / nsplit, split = (int)blockIdx.x % nsplit, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int chunk = (ntiles + nsplit - 1) / nsplit, tlo = min(split * chunk, ntiles), n_own = min(tlo + chunk, ntiles) - tlo;
  const long rowb = (long)ch * S_pad, tileb = (long)ch * (S_pad / T);
  const long khs = META ? K.head_start[ch] : 0, vhs = META ? V.head_start[ch] : 0;
  if (wave >= n_own) return;
  const int last = tlo + n_own - 1;
  ProbeRegs R0, R1;
  u32 acc = 0u;
  auto escapes = [&](ProbeRegs& R) {
    if (META) {
      const u32 rb = (u32)esc_bytes(R.kf) | ((u32)esc_bytes(R.vf) << 16), excl = row_scan16(rb) - rb;
      R.ke = load_u32x2_unaligned(K.ovf + khs + R.kto + (excl & 0xFFFFu) + (u32)esc_prefix(R.kf, 8 * (lane >> 4)));
      R.ve = load_u32x2_unaligned(V.ovf + vhs + R.vto + (excl >> 16) + (u32)esc_prefix(R.vf, 8 * (lane >> 4)));
    }
  };
  auto fold = [&](const ProbeRegs& R) { acc ^= probe_fold(R); if (META) acc ^= R.ke[0] ^ R.ke[1] ^ R.ve[0] ^ R.ve[1]; };
  probe_load<META>(K, V, rowb, tileb, khs, vhs, tlo + wave, lane, R0); escapes(R0);
  for (int i = wave; i < n_own; i += 2 * NW) {
    probe_load<META>(K, V, rowb, tileb, khs, vhs, min(tlo + i + NW, last), lane, R1); escapes(R1);
    fold(R0);
    if (i + NW >= n_own) break;
    probe_load<META>(K, V, rowb, tileb, khs, vhs, min(tlo + i + 2 * NW, last), lane, R0); escapes(R0);
    fold(R1);
  }
  if (acc == 0x9E3779B9u) sink[0] = acc;      // keeps the loads alive; practically never written
}

// The paged counterpart: the loads of k_attn_split<true, 4, ...> over a slot pool without its arithmetic.  One four-wave block per
// (batch row in `order`, kv head, split), two blocks per CU (the LDS table keeps a third one out, as registers do for the attention
// kernel); the block resolves its split's tiles (block table -> mode table) into LDS, then every wave fetches the slots of the tiles
// wave, wave + 4, ... one tile ahead: payload, tag word and eight escape bytes per lane of the K slot and of the V slot.  Tiles with a
// raw side are skipped.
constexpr int PROBE_CHUNK = 1024, SLOT_CD_ = TILE_SM, SLOT_FL_ = TILE_SM + TILE_CD, SLOT_OV_ = SLOT_FL_ + 4 * T;
struct SlotRegs { Payload k, v; u32 kf, vf; u32x2 ke, ve; };
__device__ __forceinline__ void slot_load(const uint8_t* pool, size_t TS, int2 e, int lane, SlotRegs& R) {
  const uint8_t* ks = pool + (size_t)e.x * TS; const uint8_t* vs = pool + (size_t)e.y * TS;
  load_payload(ks, ks + SLOT_CD_, lane, R.k);
  load_payload(vs, vs + SLOT_CD_, lane, R.v);
  R.kf = (u32)__builtin_nontemporal_load(reinterpret_cast<const int*>(ks + SLOT_FL_) + (lane & 15));
  R.vf = (u32)__builtin_nontemporal_load(reinterpret_cast<const int*>(vs + SLOT_FL_) + (lane & 15));
}
__device__ __forceinline__ void slot_escapes(const uint8_t* pool, size_t TS, int2 e, int lane, SlotRegs& R) {
  const u32 rb = (u32)esc_bytes(R.kf) | ((u32)esc_bytes(R.vf) << 16), excl = row_scan16(rb) - rb;
  const u32 lim = (u32)TS - (u32)SLOT_OV_ - 8u;
  R.ke = load_u32x2_unaligned(pool + (size_t)e.x * TS + SLOT_OV_ + min((excl & 0xFFFFu) + (u32)esc_prefix(R.kf, 8 * (lane >> 4)), lim));
  R.ve = load_u32x2_unaligned(pool + (size_t)e.y * TS + SLOT_OV_ + min((excl >> 16) + (u32)esc_prefix(R.vf, 8 * (lane >> 4)), lim));
}
__global__ void __launch_bounds__(256, 2) k_read_probe_paged(const uint8_t* __restrict__ pool, int TS, const int* __restrict__ mt, const int* __restrict__ bt,
                                                             int bt_stride, const int* __restrict__ seq_lens, const int* __restrict__ order, int n_kv,
                                                             int nsplit, u32* __restrict__ sink) {
  constexpr int NW = 4, NT = 256;
  __shared__ int2 table[PROBE_CHUNK];
  __shared__ u32 pad[(60 * 1024 - PROBE_CHUNK * 8) / 4];      // the attention kernel's LDS footprint: two blocks per CU
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int bh = (int)blockIdx.x / nsplit, split = ((int)blockIdx.x + bh) % nsplit, b = order[bh / n_kv], kvh = bh % n_kv;
  const int S = max(seq_lens[b], 0), ntiles = S / T, chunk = ((S + T - 1) / T + nsplit - 1) / nsplit;
  const int tlo = min(split * chunk, ntiles), thi = min(tlo + chunk, ntiles);
  u32 acc = 0u;
  if (tid == 0) pad[blockIdx.x & 1023] = 0u;
  for (int c0 = tlo; c0 < thi; c0 += PROBE_CHUNK) {
    const int n = min(PROBE_CHUNK, thi - c0);
    __syncthreads();
    for (int i = tid; i < n; i += NT) {
      const long pc = (long)bt[(long)b * bt_stride + c0 + i] * (2 * n_kv) + 2 * kvh;
      table[i] = int2{mt[pc], mt[pc + 1]};
    }
    __syncthreads();
    if (wave >= n) continue;
    SlotRegs R0, R1;
    auto fold = [&](const SlotRegs& R, int2 e) {
      if ((e.x | e.y) >= 0) acc ^= R.k.s0[0] ^ R.k.s0[3] ^ R.k.s1[1] ^ R.k.s1[2] ^ R.k.c0 ^ R.k.c1 ^ R.k.c2 ^ R.v.s0[0] ^ R.v.s0[3] ^ R.v.s1[1] ^ R.v.s1[2] ^
                                   R.v.c0 ^ R.v.c1 ^ R.v.c2 ^ R.ke[0] ^ R.ke[1] ^ R.ve[0] ^ R.ve[1];
    };
    auto entry = [&](int i) { int2 e = table[min(i, n - 1)]; if ((e.x | e.y) < 0) e = int2{max(e.x, 0), max(e.y, 0)}; return e; };      // raw side: some valid slot, not folded
    int2 e0 = entry(wave), e1;
    slot_load(pool, (size_t)TS, e0, lane, R0); slot_escapes(pool, (size_t)TS, e0, lane, R0);
    for (int i = wave; i < n; i += 2 * NW) {
      e1 = entry(i + NW); slot_load(pool, (size_t)TS, e1, lane, R1); slot_escapes(pool, (size_t)TS, e1, lane, R1);
      fold(R0, table[i]);
      if (i + NW >= n) break;
      e0 = entry(i + 2 * NW); slot_load(pool, (size_t)TS, e0, lane, R0); slot_escapes(pool, (size_t)TS, e0, lane, R0);
      fold(R1, table[i + NW]);
    }
  }
  if (acc == 0x9E3779B9u) sink[0] = acc + pad[0];
}

__global__ void __launch_bounds__(256) k_stream_copy(const u32x4* __restrict__ src, u32x4* __restrict__ dst, long n16) {
  for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n16; i += (long)gridDim.x * 256) dst[i] = src[i];
}

}  // namespace gaac

using namespace gaac;

// both return 0, -1 for rejected arguments, or the hipError_t of a failed launch
extern "C" int gaac_stream_copy(const void* src, void* dst, long nbytes, void* stream) {
  if (!src || !dst || nbytes <= 0 || nbytes % 16 != 0) return -1;
  const long n16 = nbytes / 16;
  const int blocks = (int)((n16 + 255) / 256 < 8192 ? (n16 + 255) / 256 : 8192);
  hipLaunchKernelGGL(k_stream_copy, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const u32x4*)src, (u32x4*)dst, n16);
  return (int)hipGetLastError();
}

extern "C" int gaac_read_probe(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv,
    int H, int S, int S_pad, int nsplit, int with_meta, unsigned int* sink, void* stream) {
  if (!(smk && ck && fk && tok && ovk && ohsk && smv && cv && fv && tov && ovv && ohsv && sink)) return -1;
  if (!(H > 0 && S > 0 && S % T == 0 && S <= S_pad && S_pad % T == 0 && nsplit >= 1)) return -1;
  const ProbeView K{smk, ck, fk, tok, ovk, ohsk}, V{smv, cv, fv, tov, ovv, ohsv};
  if (with_meta) hipLaunchKernelGGL(k_read_probe<true>, dim3(H * nsplit), dim3(512), 0, (hipStream_t)stream, K, V, S_pad, S / T, nsplit, sink);
  else hipLaunchKernelGGL(k_read_probe<false>, dim3(H * nsplit), dim3(512), 0, (hipStream_t)stream, K, V, S_pad, S / T, nsplit, sink);
  return (int)hipGetLastError();
}

extern "C" int gaac_read_probe_paged(const uint8_t* pool, int TS, const int* mt, const int* bt, int bt_stride, const int* seq_lens, const int* order,
                                     int B, int n_kv, int nsplit, unsigned int* sink, void* stream) {
  if (!(pool && mt && bt && seq_lens && order && sink) || B <= 0 || n_kv <= 0 || nsplit < 1 || TS < SLOT_OV_ + 16 || bt_stride <= 0) return -1;
  hipLaunchKernelGGL(k_read_probe_paged, dim3(B * n_kv * nsplit), dim3(256), 0, (hipStream_t)stream, pool, TS, mt, bt, bt_stride, seq_lens, order, n_kv,
                     nsplit, sink);
  return (int)hipGetLastError();
}
