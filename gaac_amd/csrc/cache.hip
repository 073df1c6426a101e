// Decode-step append of the compressed KV cache: one new token per (batch row, kv head) goes to the head's raw BF16 tail; the
// step that fills the 16th tail row compresses the tile in place and appends its escape bytes to the head's escape stream.
// State machine and buffers follow /root/reference/gaac/kv_cache.py:22-96 (_append_one, _append_kv, _advance) and :99-111
// (_Store); one launch does what the reference does in two (a block owns BOTH kinds of its head, so the shared counters are
// advanced after both waves are done).  No host synchronisation; safe to capture in a HIP graph.
#include "gaac_tile.h"
#include "gaac_capi.h"

namespace gaac {

struct CacheStore {      // one kind of the cache (kv_cache.py:99-111)
  u16* tail; const uint8_t* base3; const uint8_t* base4;
  uint8_t* sm; uint8_t* cd; int* flags; uint8_t* ovf; int* tile_off; int* ovf_used;
};
struct AppendArgs {
  CacheStore k, v;
  const u16* kx; const u16* vx;      // [B, n_kv, D] new tokens
  const int* slots; int* tail_len; int* S;
  int cap, ovf_cap, n_kv, NB;
  int* err;                          // bit 0: a head was full (token dropped); bit 1: an escape stream was full (tile zero-tagged)
};

template <int KIND>
__device__ __forceinline__ void append_one(const CacheStore& st, const u16* __restrict__ xrow, EncodeLds& L, int h, int pos, int Sh,
                                           const AppendArgs& A, int lane) {
  u16* tail_h = st.tail + (long)h * T * D;
  if (lane < 16) *reinterpret_cast<u32x4*>(tail_h + pos * D + 8 * lane) = *reinterpret_cast<const u32x4*>(xrow + 8 * lane);
  if (pos + 1 != T) return;
  const int tile = Sh / T;
  if ((tile + 1) * T > A.cap) { if (lane == 0) atomicOr(A.err, 1); return; }
  // rows 0..14 come from the tail as earlier steps left it, row 15 is the new token
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
    const u16* src = row < T - 1 ? tail_h + row * D : xrow;
    *reinterpret_cast<u32x4*>(&L.x[row * XROW + c16 * 8]) = *reinterpret_cast<const u32x4*>(src + c16 * 8);
  }
  const int brow = h % A.NB;
  stage_bases(L, st.base3 + (long)brow * D, st.base4 + (long)brow * D, lane);
  wave_lds_sync();
  BaseRegs Bs;
  load_base_regs<KIND>(L, lane & 15, lane >> 4, Bs);
  const long row0 = (long)h * A.cap + (long)tile * T;
  uint8_t* sm_tile = st.sm + row0 * D; uint8_t* cd_tile = st.cd + row0 * CB; int* fl_tile = st.flags + row0;
  const int used = st.ovf_used[h];
  uint8_t* dst = st.ovf + (long)h * A.ovf_cap + used;
  int total; bool fits = true;
  if (used + TILE_MAX_ESC + 8 <= A.ovf_cap) total = encode_staged_tile<KIND>(L, Bs, T, lane, sm_tile, cd_tile, fl_tile, dst);
  else {      // less than one worst-case tile of room: count first, write only what fits
    total = encode_staged_tile<KIND>(L, Bs, T, lane, sm_tile, cd_tile, fl_tile, nullptr);
    fits = used + total + 8 <= A.ovf_cap;
    if (fits) encode_staged_tile<KIND>(L, Bs, T, lane, sm_tile, cd_tile, fl_tile, dst);
  }
  if (fits) {
    if (lane == 0) { st.tile_off[(long)h * (A.cap / T) + tile] = used; st.ovf_used[h] = used + total; }
  } else {    // keep every later reader in bounds: the tile reads as all tier 0 (wrong values, flagged)
    if (lane < T) fl_tile[lane] = 0;
    if (lane == 0) { st.tile_off[(long)h * (A.cap / T) + tile] = 0; atomicOr(A.err, 2); }
  }
}

// grid (B*n_kv), 128 threads: wave 0 = K, wave 1 = V of cache head SLOT[b]*n_kv + kvh
__global__ void __launch_bounds__(128) k_cache_append(const AppendArgs A) {
  __shared__ EncodeLds L[2];
  const int i = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int slot = A.slots[i / A.n_kv];
  if (slot < 0) return;
  const int h = slot * A.n_kv + i % A.n_kv;
  const int pos = A.tail_len[h], Sh = A.S[h];
  if (wave == 0) append_one<KIND_K>(A.k, A.kx + (long)i * D, L[0], h, pos, Sh, A, lane);
  else append_one<KIND_V>(A.v, A.vx + (long)i * D, L[1], h, pos, Sh, A, lane);
  __syncthreads();
  if (tid == 0) {      // _advance (kv_cache.py:86-96)
    const bool full = pos + 1 == T;
    A.tail_len[h] = full ? 0 : pos + 1;
    if (full && Sh + T <= A.cap) A.S[h] = Sh + T;
  }
}

}  // namespace gaac

using namespace gaac;

extern "C" int gaac_cache_append(
    const int* slots, int B, int n_kv, const void* k_new, const void* v_new, int* tail_len, int* S, int cap, int ovf_cap, int NB,
    void* k_tail, const uint8_t* k_base3, const uint8_t* k_base4, uint8_t* k_sm, uint8_t* k_codes, int* k_flags, uint8_t* k_ovf, int* k_tile_off, int* k_ovf_used,
    void* v_tail, const uint8_t* v_base3, const uint8_t* v_base4, uint8_t* v_sm, uint8_t* v_codes, int* v_flags, uint8_t* v_ovf, int* v_tile_off, int* v_ovf_used,
    int* err, void* stream) {
  GAAC_REQUIRE(slots && k_new && v_new && tail_len && S && err, "gaac_cache_append: null pointer");
  GAAC_REQUIRE(k_tail && k_base3 && k_base4 && k_sm && k_codes && k_flags && k_ovf && k_tile_off && k_ovf_used, "gaac_cache_append: null K store pointer");
  GAAC_REQUIRE(v_tail && v_base3 && v_base4 && v_sm && v_codes && v_flags && v_ovf && v_tile_off && v_ovf_used, "gaac_cache_append: null V store pointer");
  GAAC_REQUIRE(B > 0 && n_kv > 0 && NB > 0 && cap > 0 && cap % T == 0 && ovf_cap >= 8, "gaac_cache_append: bad sizes B=%d n_kv=%d NB=%d cap=%d ovf_cap=%d", B, n_kv, NB, cap, ovf_cap);
  AppendArgs A;
  A.k = CacheStore{(u16*)k_tail, k_base3, k_base4, k_sm, k_codes, k_flags, k_ovf, k_tile_off, k_ovf_used};
  A.v = CacheStore{(u16*)v_tail, v_base3, v_base4, v_sm, v_codes, v_flags, v_ovf, v_tile_off, v_ovf_used};
  A.kx = (const u16*)k_new; A.vx = (const u16*)v_new; A.slots = slots; A.tail_len = tail_len; A.S = S;
  A.cap = cap; A.ovf_cap = ovf_cap; A.n_kv = n_kv; A.NB = NB; A.err = err;
  hipLaunchKernelGGL(k_cache_append, dim3(B * n_kv), dim3(128), 0, (hipStream_t)stream, A);
  return launch_status("gaac_cache_append");
}
