// Fused split-K decode attention over compressed K/V for gfx950 (wave64, MFMA), the raw-BF16 tail, and the split merge.
// Counterpart of gaac_attn / gaac_tail / gaac_combine / gaac_attn_launch in /root/reference/gaac/kernel.py:48-326
// (same inputs, same partial (m, l, acc) protocol, same slot map and padded-row behaviour), redesigned for CDNA4:
//
//   * one block = (batch row, kv head, split), 8 waves (one block per CU) for launches of up to 256 blocks, else 4 waves (two per CU);
//     the waves of a block take their tiles from a counter in LDS (the two waves sharing a SIMD would otherwise finish far apart);
//   * scores   S[16 tok x 16 heads]  = K[16 x 128] . Q^T      : 4 x v_mfma_f32_16x16x32_bf16   (A = decoded K units)
//   * output   O^T[128 x 16 heads]  += V^T[128 x 16] . P^T     : 8 x v_mfma_f32_16x16x16_bf16   (A = decoded V units)
//     The score tile lands in the register layout the second product wants for P^T, so P never crosses lanes.
//   * the GQA group (<= 16 query heads) rides in the N dimension; register use does not depend on it;
//   * three-stage prefetch per wave: tag words two tiles ahead, payload + escape bytes one tile ahead, consume;
//   * the raw BF16 tail of a cache head (<= 16 tokens) is attended by one wave of the block that owns the last split, as an extra
//     partial of that block's merge; the wave then joins the tile hand-out, so the other waves absorb the tiles it did not take;
//   * the last block of a (row, kv head) to publish its partial merges all of them (fused gaac_combine); k_attn_combine is the
//     two-launch alternative;
//   * k_attn_split<true, .> reads the paged slot pool through block and mode tables (paged_kernel.py:42-241).
//   Softmax runs in base 2 (scale * log2 e folded into the scores).
#include <atomic>
#include <mutex>
#include "gaac_tile.h"
#include "gaac_capi.h"
#include "../../include/gaac_hip.h"

// GAAC_WAVES12 (python -m gaac_amd.build --waves12 -> libgaac_hip_w12.so) is a measurement build, not the product: launches of up to
// 256 blocks over contiguous stores with host lengths run twelve-wave blocks, three waves per SIMD instead of two.  The register cap
// falls from 256 to 168 per lane; to get under it without spilling the tile loop, this build reads the query words from LDS for every
// score product instead of keeping them in 16 registers, and looks up the V side's escape and base words after the score products
// instead of together with the K side's.  Both cost time at two waves per SIMD, which is why the product does neither.
#ifdef GAAC_WAVES12
constexpr bool WAVES12 = true;
#else
constexpr bool WAVES12 = false;
#endif

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
  u32* epochs; u16* out;       // fused merge: [0] the epoch of the last merged launch, [1] failure bits, [2 + i] arrival mark of block i; pm / pl / pa then hold 64-bit records
  int S_all;                   // >= 0: every addressed cache head holds exactly S_all compressed tokens (sl is not read)
  // paged slot pool (k_attn_split<true>): sl = tokens per batch row, bt = block table [B][bt_stride], mt = mode table, pool = tile
  // slots of TS bytes, raw = side pool of BF16 tiles; physical tile = block*2*n_kv + 2*kvh + kind
  const uint8_t* pool; const u16* raw; const int* mt; const int* bt; int bt_stride; int TS;
  // paged: raw tiles queued by the preceding store (gaac_paged_store's freeq) that this launch pushes back onto the free stack (or null)
  const int* freeq; int n_free; int* stack; int* top;
#ifdef GAAC_PHASE_TIMING
  long long* dbg;
#endif
};
#ifdef GAAC_PHASE_TIMING
#define GAAC_STAMP(k) do { if (A.dbg && threadIdx.x == 0) A.dbg[(long)blockIdx.x * 8 + (k)] = wall_clock64(); } while (0)
#define GAAC_MSTAMP(k, v) do { if (A.dbg && threadIdx.x == 0) A.dbg[(2 * (long)gridDim.x + blockIdx.x) * 8 + (k)] = (v); } while (0)
#else
#define GAAC_STAMP(k) do {} while (0)
#define GAAC_MSTAMP(k, v) do {} while (0)
#endif
constexpr int MAX_CHUNK = 1024;  // tiles whose slot lookups a block keeps in LDS at a time (paged mode); longer splits go on in further rounds
constexpr int SLOT_CD = TILE_SM, SLOT_FL = TILE_SM + TILE_CD, SLOT_OV = SLOT_FL + 4 * T;      // byte offsets inside a tile slot

__device__ __forceinline__ float bf16_bits_to_float(u32 h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ u32 pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  bf16x2 v; v[0] = (__bf16)lo; v[1] = (__bf16)hi;
  return __builtin_bit_cast(u32, v);
}

// ---------------------------------------------------------------------------------------------------- fused merge
// Merge of the split partials (gaac_combine, /root/reference/gaac/kernel.py:281-294) inside the split kernel, by ONE block of each
// (batch row, kv head), without atomics and without any block waiting for a store acknowledgement on its way out:
//
//   * One word, epochs[0], holds the epoch of the last merged launch.  Every block reads it while its first tiles are in flight; this
//     launch's EPOCH is that value + 1 (skipping 0 when the 32-bit counter wraps), the same for all blocks: the word is advanced by
//     the last block of the grid, as its very last action, and only after it has SEEN the arrival mark of every block of the grid
//     (epochs[2 + block], stored by the block once its first wave is through its tiles: a block that has marked has read the word
//     long ago; blocks of a grid larger than the GPU holds start whenever a CU of their XCD frees up, in no order the other XCDs
//     know of).
//     A record slot read by a launch was last written by an earlier launch, whatever its shape, under another epoch (the same
//     value returns only after 2^32 - 1 launches on the same records), or never, and then holds the unused epoch 0.
//   * A partial value travels as one 64-bit record (fp32 bits | epoch << 32) written with a single 64-bit store: a reader sees either
//     the whole record of this launch or an older one, never a torn one (naturally aligned 64-bit accesses are single-copy atomic),
//     so no fence, flag or acknowledgement orders data against a separate signal.  Records are written with agent-scope stores
//     (write-through) and read with agent-scope loads (they bypass the reader's L2): the blocks of a head sit on different XCDs.
//   * The MERGERS are the head's last (up to sixteen) blocks in index order; each takes a share of the head's output (half a query head
//     per wave), because one CU pulls records at only ~80 GB/s.  Once a merger has stored its own partial it loads the records of its
//     share from all blocks of the head and re-reads those whose epoch is not yet the launch's.  Everything a merger waits for is
//     running, done, or one of the at most fifteen later mergers of the same head, which wait for nobody but each other's stores,
//     and those precede every wait.  The wait is bounded all the same (MERGE_SPIN_LIMIT re-reads): a merger that gives up writes its
//     rows as NaN and sets bit 0 of epochs[1]; the grid's last block sets bit 1 if it gives up waiting for the other blocks (it then
//     leaves the epoch word alone).  The owner of the workspace polls epochs[1] and re-arms after a failure.
//   * Launches that share the records and the epoch words must be ordered on one stream.  To re-arm after a failed launch, zero all.
typedef __attribute__((ext_vector_type(4))) float f32x4v;
__device__ __forceinline__ void store_partial(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ void ll_store(u64* p, float v, u32 epoch) {
  __hip_atomic_store(p, (u64)__float_as_uint(v) | ((u64)epoch << 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ u64 ll_load(const u64* p) { return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ bool ll_stale(u64 r, u32 epoch) { return (u32)(r >> 32) != epoch; }
__device__ __forceinline__ float ll_value(u64 r) { return __uint_as_float((u32)r); }
constexpr int MERGE_SPIN_LIMIT = 1 << 16;      // re-reads of a chunk before the merger gives up (each with a short sleep: ~0.1 s)
// (no branch around the load: a load under a branch is waited for where the branch ends, together with everything issued before it)
__device__ __forceinline__ u32 load_epoch(const AttnArgs& A, int bh) {
  const u32* p = A.epochs ? A.epochs : reinterpret_cast<const u32*>(A.q);
  const u32 e = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return e + 1u + (e == 0xFFFFFFFFu ? 1u : 0u);      // epoch 0 is never used: zeroed records stay stale when the counter wraps
}
// A block barrier that orders LDS traffic only.  (__syncthreads() also waits for the block's global stores to be acknowledged,
// which for write-through stores is a trip to memory.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// LDS of a merging block: per wave the (m, then weight) and l of every slot.
template <int NW> struct MergeScratch { float f[NW][MAX_SLOTS], l[NW][MAX_SLOTS]; };

// One merger's work for half a query head (64 output channels), shared by the NW waves of the block.  A wave owns 64 / NW channels
// and sums them over ALL slots, so the waves exchange nothing and no block barrier lies between the records' arrival and the
// output: lane (g, c) = (lane / CPW, lane % CPW) reads the accumulator records of channel c of the wave for the slots g, g + SG, ...
// (SG = 64 / CPW slot groups); the groups' sums meet through DPP.  Every wave reads the m / l records of all slots (lane = slot)
// and derives the slots' weights itself.  Called by all threads of the block.
__device__ __forceinline__ void merge_failed(const AttnArgs& A, u32 bit) {
  __hip_atomic_fetch_or(A.epochs + 1, bit, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <int NW>
__device__ __forceinline__ void merge_half_head(const AttnArgs& A, long row, int half, u32 epoch, MergeScratch<NW>& X, int wave, int lane) {
  constexpr int CPW = 64 / NW, SG = 64 / CPW;      // channels per wave (8 | 16), slot groups (8 | 4)
  constexpr int CH = 8;                             // accumulator records in flight per lane: one round for up to CH * SG splits
  const int nslot = A.nslot, g = lane / CPW, d = 64 * half + CPW * wave + lane % CPW;
  const u64* rm = reinterpret_cast<const u64*>(A.pm) + row * nslot;
  const u64* rl = reinterpret_cast<const u64*>(A.pl) + row * nslot;
  const u64* ra = reinterpret_cast<const u64*>(A.pa) + row * nslot * D + d;
  float* fs = X.f[wave]; float* ls = X.l[wave];
  bool ok = true;
  // all loads of the first round are issued before the first use, none under a branch (a slot past the end reads the last slot
  // instead and is ignored): the lane's first CH accumulator records ...
  u64 v[CH];
#pragma unroll
  for (int k = 0; k < CH; ++k) v[k] = ll_load(ra + (long)min(g + SG * k, nslot - 1) * D);
  // ... then m / l of slots 0..63 (one slot per lane); everything is re-read together until it carries this launch's epoch
  u64 mr = ll_load(rm + min(lane, nslot - 1)), lr = ll_load(rl + min(lane, nslot - 1));
  GAAC_MSTAMP(0, wall_clock64());
  for (int spin = 0;; ++spin) {
    bool stale = lane < nslot && (ll_stale(mr, epoch) || ll_stale(lr, epoch));
#pragma unroll
    for (int k = 0; k < CH; ++k) stale |= g + SG * k < nslot && ll_stale(v[k], epoch);
    if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
    if (spin >= MERGE_SPIN_LIMIT) { ok = false; break; }
    __builtin_amdgcn_s_sleep(1);
    if (lane < nslot && ll_stale(mr, epoch)) mr = ll_load(rm + lane);
    if (lane < nslot && ll_stale(lr, epoch)) lr = ll_load(rl + lane);
#pragma unroll
    for (int k = 0; k < CH; ++k) { const int s = g + SG * k; if (s < nslot && ll_stale(v[k], epoch)) v[k] = ll_load(ra + (long)s * D); }
  }
  GAAC_MSTAMP(1, wall_clock64());
  const float m_own = lane < nslot ? ll_value(mr) : -INFINITY, l_own = lane < nslot ? ll_value(lr) : 0.f;      // slot = lane
  float m = m_own;
  for (int s0 = 64; ok && s0 < nslot; s0 += 64) {      // more than 64 splits: the other m / l records, kept in LDS
    const int s = s0 + lane;
    mr = s < nslot ? ll_load(rm + s) : 0ull; lr = s < nslot ? ll_load(rl + s) : 0ull;
    for (int spin = 0; __builtin_amdgcn_ballot_w64(s < nslot && (ll_stale(mr, epoch) || ll_stale(lr, epoch))) != 0; ++spin) {
      if (spin >= MERGE_SPIN_LIMIT) { ok = false; break; }
      __builtin_amdgcn_s_sleep(1);
      if (s < nslot && ll_stale(mr, epoch)) mr = ll_load(rm + s);
      if (s < nslot && ll_stale(lr, epoch)) lr = ll_load(rl + s);
    }
    if (s < nslot) { fs[s] = ll_value(mr); ls[s] = ll_value(lr); m = fmaxf(m, ll_value(mr)); }
  }
  const float mx = wave_max(m);
  // the slots' weights go to LDS for the lanes that need them (the wave's own region: no block barrier)
  const float f_own = m_own != -INFINITY ? __builtin_amdgcn_exp2f(m_own - mx) : 0.f;
  float l = l_own * f_own;
  fs[lane] = f_own;
  for (int s = lane + 64; s < nslot; s += 64) {      // each lane revisits the slots it wrote
    const float pmv = fs[s], f = pmv != -INFINITY ? __builtin_amdgcn_exp2f(pmv - mx) : 0.f;
    fs[s] = f; l += ls[s] * f;
  }
  l = wave_sum(l);
  wave_lds_sync();
  float acc = 0.f;
  for (int s0 = g; s0 < nslot; s0 += SG * CH) {
    if (s0 != g) {      // more than CH * SG splits: the lane's further records
#pragma unroll
      for (int k = 0; k < CH; ++k) { const int s = s0 + SG * k; v[k] = s < nslot ? ll_load(ra + (long)s * D) : 0ull; }
      for (int spin = 0; ok; ++spin) {
        bool stale = false;
#pragma unroll
        for (int k = 0; k < CH; ++k) stale |= s0 + SG * k < nslot && ll_stale(v[k], epoch);
        if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
        if (spin >= MERGE_SPIN_LIMIT) { ok = false; break; }
        __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int k = 0; k < CH; ++k) { const int s = s0 + SG * k; if (s < nslot && ll_stale(v[k], epoch)) v[k] = ll_load(ra + (long)s * D); }
      }
    }
#pragma unroll
    for (int k = 0; k < CH; ++k) {
      const int s = s0 + SG * k;
      if (s < nslot) { const float f = fs[s]; acc += f != 0.f ? ll_value(v[k]) * f : 0.f; }      // an empty partial's accumulator may hold anything
    }
  }
  // the slot groups' sums of a channel sit CPW lanes apart: across the four 16-lane rows, and for CPW = 8 also 8 lanes apart in a row
  acc = quad_rows_sum(acc);
  if (CPW == 8) acc += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, acc), 0x128 /* row_ror:8 */, 0xF, 0xF, false));
  GAAC_MSTAMP(2, wall_clock64());
  ok = __builtin_amdgcn_ballot_w64(!ok) == 0;
  if (!ok && lane == 0) merge_failed(A, 1u);
  if (lane < CPW) {
    const float o = ok ? (l > 0.f ? acc / l : 0.f) : __builtin_nanf("");
    A.out[row * D + d] = __builtin_bit_cast(u16, (__bf16)o);
  }
  GAAC_MSTAMP(4, wall_clock64());
  wave_lds_sync();      // the wave's LDS region is free for its next item
}
// The merge of a head is shared by its last `mergers` blocks in index order (merge_ranks): the block of rank j takes the half heads
// j, j + mergers, ..., so that no single CU has to pull all the records.  Called by all threads of a merging block after its own
// partial has been stored and every thread is done with the LDS that X aliases.
__device__ __forceinline__ int merge_ranks(int G, int nslot) { return min(min(16, 2 * G), nslot); }
// Arrival marks: epochs[2 + i] = the epoch block i of the grid works under, stored by the block's first wave when it leaves its tile
// loop (long after it read the epoch word, well before the block publishes its partial).  The grid's last block reads all marks
// before it advances the epoch word.
constexpr int EPOCH_WORDS = 2;      // words of the epoch buffer ahead of the arrival marks
__device__ __forceinline__ void mark_arrival(const AttnArgs& A, u32 epoch) {
  __hip_atomic_store(A.epochs + EPOCH_WORDS + blockIdx.x, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <int NWB>      // NWB: waves of the block; twelve-wave blocks (measurement build) merge with their first eight waves
__device__ __forceinline__ void merge_heads(const AttnArgs& A, long qh0, int G, u32 epoch, int rank, int mergers, int tid, MergeScratch<(NWB > 8 ? 8 : NWB)>& X) {
  constexpr int NW = NWB > 8 ? 8 : NWB;
  const int wave = tid >> 6, lane = tid & 63;
  if (NWB > NW && wave >= NW) { if (blockIdx.x == gridDim.x - 1) lds_barrier(); return; }      // (the last block meets once more below)
  const bool last = blockIdx.x == gridDim.x - 1;
  // The last block of the grid advances the epoch word for the next launch, once every block of this launch has marked its arrival
  // (and so has read the word).  The marks' first read is issued here, ahead of the merge work, and looked at after it: by then the
  // other blocks have long left their loops, so the check normally costs no trip to memory of its own.
  constexpr int XK = 2048 / (64 * NW);      // marks per lane held in registers: the first 2048 blocks of the grid
  const u32* marks = A.epochs + EPOCH_WORDS;
  const int nblocks = (int)gridDim.x, xi = 64 * wave + lane;
  u32 xm[XK];
  if (last) {
#pragma unroll
    for (int k = 0; k < XK; ++k) xm[k] = __hip_atomic_load(marks + min(xi + 64 * NW * k, nblocks - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  // The first item stands outside the loop: at a loop header the compiler waits for every memory operation in flight, which here
  // would be the acknowledgement of the block's own record stores (a round trip to memory) before the first record load is issued.
  int item = rank;
  if (item < 2 * G) { merge_half_head<NW>(A, qh0 + (item >> 1), item & 1, epoch, X, wave, lane); item += mergers; }
  for (; item < 2 * G; item += mergers) merge_half_head<NW>(A, qh0 + (item >> 1), item & 1, epoch, X, wave, lane);
  if (!last) return;
  bool grid_ok = true;
  for (int spin = 0;; ++spin) {
    bool stale = false;
#pragma unroll
    for (int k = 0; k < XK; ++k) stale |= xm[k] != epoch;
    if (__builtin_amdgcn_ballot_w64(stale) == 0) break;
    if (spin >= MERGE_SPIN_LIMIT) { grid_ok = false; break; }
    __builtin_amdgcn_s_sleep(1);
#pragma unroll
    for (int k = 0; k < XK; ++k)
      if (xm[k] != epoch) xm[k] = __hip_atomic_load(marks + min(xi + 64 * NW * k, nblocks - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  for (int i0 = 2048; grid_ok && i0 < nblocks; i0 += 64 * NW) {      // grids beyond 2048 blocks: the remaining marks, a round at a time
    const int i = min(i0 + xi, nblocks - 1);
    for (int spin = 0; __builtin_amdgcn_ballot_w64(__hip_atomic_load(marks + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != epoch) != 0; ++spin) {
      if (spin >= MERGE_SPIN_LIMIT) { grid_ok = false; break; }
      __builtin_amdgcn_s_sleep(1);
    }
  }
  // The waves' verdicts meet in LDS behind a barrier that orders LDS traffic only: a full block barrier would first wait for the
  // acknowledgement of the output rows just stored, and the epoch store would then be a second trip to memory at the launch's very end.
  grid_ok = __builtin_amdgcn_ballot_w64(!grid_ok) == 0;
  if (lane == 0) X.l[wave][0] = grid_ok ? 1.f : 0.f;
  lds_barrier();
  if (tid == 0) {
    bool all = true;
#pragma unroll
    for (int w = 0; w < NW; ++w) all &= X.l[w][0] != 0.f;
    if (all) __hip_atomic_store(A.epochs, epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else merge_failed(A, 2u);
  }
}

// ---------------------------------------------------------------------------------------------------- uncompressed rows
// Attention of the block's G query heads over up to 16 rows kept as plain BF16 (the raw tail of a cache head, gaac_tail of
// /root/reference/gaac/kernel.py:220-279), done by the block's first 256 threads in fp32 on the VALU (all threads take part in the barriers).  The result is folded into the running
// partial (m, l, acc) that the block merge treats as a fifth wave; several calls accumulate (online softmax).
struct RawScratch {              // lives in the block-merge buffer, which is idle until the waves have finished their tiles
  float qs[GMAX][D];             // the query heads in fp32, natural channel order
  float sc[GMAX][T];             // scores, then probabilities
  float alpha[GMAX];             // rescale factor of the running partial
  u16 krows[T * D], vrows[T * D];   // a compressed tile decoded next to a raw one (paged mode: only one kind of a tile is raw)
};
template <int NT>
__device__ __forceinline__ void raw_rows_begin(RawScratch& R, const AttnArgs& A, long qh0, int G, int tid) {
  for (int i = tid; i < G * D; i += NT) R.qs[i >> 7][i & 127] = bf16_bits_to_float(A.q[qh0 * D + i]);
}
// krows / vrows: 16 x 128 BF16, row stride D; rows >= nvalid are ignored.  m5/l5/acc5: the running partial [GMAX], [GMAX], [GMAX][D].
template <int NT>
__device__ __forceinline__ void raw_rows_attend(RawScratch& R, const u16* __restrict__ krows, const u16* __restrict__ vrows, int nvalid,
                                                float scale_log2e, int G, int tid, float* __restrict__ m5, float* __restrict__ l5,
                                                float (*__restrict__ acc5)[D]) {
  __syncthreads();               // qs is filled / the previous call is done with sc
  const int t = tid >> 4, c = tid & 15;
  // all global loads of the call up front (one memory latency): this thread's piece of a K row, and for the output the two
  // channels 2 (tid & 63), +1 of all 16 V rows
  u32x4 kv = {0u, 0u, 0u, 0u};
  if (t < nvalid && t < T) kv = *reinterpret_cast<const u32x4*>(krows + t * D + 8 * c);
  u32 vv[T];
#pragma unroll
  for (int tk = 0; tk < T; ++tk) vv[tk] = *reinterpret_cast<const u32*>(vrows + min(tk, max(nvalid - 1, 0)) * D + 2 * (tid & 63));
#pragma unroll
  for (int tk = 0; tk < T; ++tk) vv[tk] = tk < nvalid ? vv[tk] : 0u;      // rows past the end weigh 0: keep an Inf of the clamped row out of 0 * Inf
  float kr[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) { kr[2 * i] = bf16_bits_to_float(kv[i] & 0xFFFFu); kr[2 * i + 1] = bf16_bits_to_float(kv[i] >> 16); }
  for (int g = 0; g < G; ++g) {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) d += R.qs[g][8 * c + i] * kr[i];
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) d += __shfl_xor(d, o, 16);
    if (c == 0 && t < T) R.sc[g][t] = t < nvalid ? d * scale_log2e : -INFINITY;
  }
  __syncthreads();
  {   // thread (g = tid >> 4, token = tid & 15): softmax over the 16 lanes of the row, merged into the running partial
    const int g = tid >> 4, tk = tid & 15;
    const float s = g < G ? R.sc[g][tk] : -INFINITY;
    float mt = s;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) mt = fmaxf(mt, __shfl_xor(mt, o, 16));
    const float m_old = g < G ? m5[g] : -INFINITY, m_new = fmaxf(m_old, mt), mu = m_new == -INFINITY ? 0.f : m_new;
    const float p = __builtin_amdgcn_exp2f(s - mu);        // rows >= nvalid: exp2(-inf) = 0
    float lt = p;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) lt += __shfl_xor(lt, o, 16);
    __syncthreads();
    if (g < G) {
      R.sc[g][tk] = p;
      if (tk == 0) {
        const float al = m_old == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_old - mu);
        R.alpha[g] = al; m5[g] = m_new; l5[g] = l5[g] * al + lt;
      }
    }
  }
  __syncthreads();
  const int d2 = 2 * (tid & 63);
  for (int g = tid >> 6; g < G; g += NT / 64) {
    const float al = R.alpha[g];
    float a0 = acc5[g][d2] * al, a1 = acc5[g][d2 + 1] * al;
#pragma unroll
    for (int tk = 0; tk < T; ++tk) { const float p = R.sc[g][tk]; a0 += p * bf16_bits_to_float(vv[tk] & 0xFFFFu); a1 += p * bf16_bits_to_float(vv[tk] >> 16); }
    acc5[g][d2] = a0; acc5[g][d2 + 1] = a1;
  }
}

// The same for ONE wave and rows in global memory: the raw tail of a cache head is attended by wave 0 of the block that owns the last
// split, before that wave joins the block's tile hand-out (the other waves pick up the tiles it does not get to).  No block barrier.
// Lane (t = lane >> 2, c = lane & 3) takes row t, channels 32c .. 32c+31 for the scores; lane owns output dims 2*lane, 2*lane+1.
__device__ __forceinline__ void wave_rows_attend(float (*__restrict__ sc)[T], const u16* __restrict__ krows, const u16* __restrict__ vrows,
                                                 int nvalid, const u16* __restrict__ qrows, float scale_log2e, int G, int lane,
                                                 float* __restrict__ m5, float* __restrict__ l5, float (*__restrict__ acc5)[D]) {
  const int t = lane >> 2, c = lane & 3;
  float kr[32];
  {
    u32x4 kv[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {      // no load under a branch: rows past the end read the last valid row and are zeroed
      kv[j] = *reinterpret_cast<const u32x4*>(krows + min(t, nvalid - 1) * D + 32 * c + 8 * j);
      if (t >= nvalid) kv[j] = u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) { kr[8 * j + 2 * i] = bf16_bits_to_float(kv[j][i] & 0xFFFFu); kr[8 * j + 2 * i + 1] = bf16_bits_to_float(kv[j][i] >> 16); }
  }
  for (int g = 0; g < G; ++g) {
    float d = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const u32x4 qv = *reinterpret_cast<const u32x4*>(qrows + g * D + 32 * c + 8 * j);
#pragma unroll
      for (int i = 0; i < 4; ++i) d += bf16_bits_to_float(qv[i] & 0xFFFFu) * kr[8 * j + 2 * i] + bf16_bits_to_float(qv[i] >> 16) * kr[8 * j + 2 * i + 1];
    }
    d += __shfl_xor(d, 1, 64); d += __shfl_xor(d, 2, 64);
    if (c == 0) sc[g][t] = t < nvalid ? d * scale_log2e : -INFINITY;
  }
  wave_lds_sync();
  for (int g = lane >> 4; g < G; g += 4) {      // 16 lanes per head: softmax over the row
    const int tk = lane & 15;
    const float s = sc[g][tk];
    float mt = s;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) mt = fmaxf(mt, __shfl_xor(mt, o, 16));
    const float p = __builtin_amdgcn_exp2f(s - (mt == -INFINITY ? 0.f : mt));
    float lt = p;
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) lt += __shfl_xor(lt, o, 16);
    sc[g][tk] = p;
    if (tk == 0) { m5[g] = mt; l5[g] = lt; }
  }
  wave_lds_sync();
  u32 vv[T];
#pragma unroll
  for (int tk = 0; tk < T; ++tk) vv[tk] = *reinterpret_cast<const u32*>(vrows + min(tk, nvalid - 1) * D + 2 * lane);
#pragma unroll
  for (int tk = 0; tk < T; ++tk) vv[tk] = tk < nvalid ? vv[tk] : 0u;      // rows past the end weigh 0: keep an Inf of the clamped row out of 0 * Inf
  for (int g = 0; g < G; ++g) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int tk = 0; tk < T; ++tk) { const float p = sc[g][tk]; a0 += p * bf16_bits_to_float(vv[tk] & 0xFFFFu); a1 += p * bf16_bits_to_float(vv[tk] >> 16); }
    acc5[g][2 * lane] = a0; acc5[g][2 * lane + 1] = a1;
  }
}

// ---------------------------------------------------------------------------------------------------- block tables (LDS)
// xlut[e]: the four exponent-field words carrying the 4th code bits of escape byte e (bit p -> element p, bit 4+p -> element p+4).
// sel[t]:  v_perm selector that spreads a lane's 8 prefetched escape bytes to one byte per unit, indexed by the lane's four
//          tags t (2 bits each): byte u = offset of unit u's escape byte when the unit is a 4-bit group (and the offset
//          is < 8), else 0x0C (-> 0).
// bw*:     exponent-base words [tier][group][p] of this block's kv head;  qw: the query words [head][group][p].
struct AttnLds {
  u32x4 xlut[256];
  u32 sel[256];
  u32x4 bwk[2][NG], bwv[2][NG];
  u32x4 qw[GMAX][NG];
};
// Block merge: one partial per wave plus one (index NW) for the uncompressed rows.  acc[0..3] double as RawScratch before the waves
// publish, acc[0..NW-1] as the merge factors afterwards.
template <int NW> struct MergeLds { float m[NW + 1][GMAX], l[NW + 1][GMAX]; float acc[NW + 1][GMAX][D]; };
static_assert(sizeof(RawScratch) <= 4 * GMAX * D * sizeof(float) && sizeof(MergeScratch<4>) <= 5 * GMAX * D * sizeof(float) &&
              sizeof(MergeScratch<8>) <= 9 * GMAX * D * sizeof(float), "scratch views must fit the merge buffer");
struct TableRegs { u32 b0, b1; u32 qlo[4], qhi[4]; };      // one thread's raw inputs of the per-block tables
// Global loads only, in two parts so that each can be issued as soon as its address is known (the query rows need the batch row, the
// base rows the cache head) and waited for only when the tables are written.
__device__ __forceinline__ void tables_load_q(TableRegs& Tr, int tid, const u16* __restrict__ qrows, int G) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {      // query words: head = idx >> 6, group = (idx >> 2) & 15, p = idx & 3 (heads >= G: any valid row)
    const int idx = tid + 256 * k, h = min(idx >> 6, G - 1), g = (idx >> 2) & 15, p = idx & 3;
    const u16* qp = qrows + h * D;
    Tr.qlo[k] = qp[chan_k(8 * g + p)]; Tr.qhi[k] = qp[chan_k(8 * g + p + 4)];
  }
}
__device__ __forceinline__ void tables_load_bases(TableRegs& Tr, int tid, const uint8_t* k3, const uint8_t* k4, const uint8_t* v3,
                                                  const uint8_t* v4, int brow) {
  // one base word per thread: kind = tid >> 7, tier = (tid >> 6) & 1, group = (tid >> 2) & 15, p = tid & 3
  const int kind = tid >> 7, tier = (tid >> 6) & 1, g = (tid >> 2) & 15, p = tid & 3;
  const uint8_t* row = (kind ? (tier ? v4 : v3) : (tier ? k4 : k3)) + (long)brow * D;
  const int c0 = kind ? chan_v(8 * g + p) : chan_k(8 * g + p), c1 = kind ? chan_v(8 * g + p + 4) : chan_k(8 * g + p + 4);
  Tr.b0 = row[c0]; Tr.b1 = row[c1];
}
__device__ __forceinline__ void tables_store(AttnLds& L, TableRegs Tr, int tid, int G) {
  // the loaded values are first needed HERE: keeps the compiler from packing them (and waiting for them) where they were loaded
  asm volatile("" : "+v"(Tr.b0), "+v"(Tr.b1), "+v"(Tr.qlo[0]), "+v"(Tr.qlo[1]), "+v"(Tr.qlo[2]), "+v"(Tr.qlo[3]), "+v"(Tr.qhi[0]),
               "+v"(Tr.qhi[1]), "+v"(Tr.qhi[2]), "+v"(Tr.qhi[3]));
  {
    const u32 e = (u32)tid;
    u32x4 w;
#pragma unroll
    for (int p = 0; p < 4; ++p) w[p] = (((e >> p) & 1u) << 10) | (((e >> (4 + p)) & 1u) << 26);
    L.xlut[tid] = w;
    u32 selw = 0u, off = 0u;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const u32 t = (e >> (2 * u)) & 3u;
      selw |= ((t == 1u && off < 8u) ? off : 0x0Cu) << (8 * u);
      off += (u32)tag_size(t);
    }
    L.sel[tid] = selw;
  }
  {
    const int kind = tid >> 7, tier = (tid >> 6) & 1, g = (tid >> 2) & 15, p = tid & 3;
    u32* dst = kind ? reinterpret_cast<u32*>(&L.bwv[tier][g]) : reinterpret_cast<u32*>(&L.bwk[tier][g]);
    dst[p] = (Tr.b0 << 7) | (Tr.b1 << 23);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int idx = tid + 256 * k, h = idx >> 6, g = (idx >> 2) & 15, p = idx & 3;
    reinterpret_cast<u32*>(&L.qw[h][g])[p] = h < G ? Tr.qlo[k] | (Tr.qhi[k] << 16) : 0u;
  }
}

// ---------------------------------------------------------------------------------------------------- tile loaders
struct KindRegs {                // one lane's view of one tile (K or V)
  Payload pay;
  u32 f;                         // the lane's four tags (bits 8q .. 8q+7 of the tag word of its line)
  u32 pos0;                      // offset of the lane's first unit's escape bytes: in the head's stream | in the tile (paged)
  u32x2 e;                       // the 8 escape bytes from pos0 on
};
struct TileRegs { KindRegs k, v; };
struct TagRegs { u32 kfl, vfl; u32 kto, vto; int raw; };      // kto/vto: tile offset in the head's escape stream | slot index (paged)

struct Bases {                   // uniform (scalar) views of one cache head; paged mode uses kov = vov = pool and TS only
  const uint8_t* ksm; const uint8_t* kcd; const int* kfl; const int* kto; const uint8_t* kov;
  const uint8_t* vsm; const uint8_t* vcd; const int* vfl; const int* vto; const uint8_t* vov;
  int TS;
};
struct TileTable { const int2* tt; int tlo; };      // paged mode: mode-table entries (K, V) of the block's tiles, in LDS

// start of a tile's escape bytes
template <bool PAGED>
__device__ __forceinline__ const uint8_t* esc_of_tile(const uint8_t* ov, u32 to, int TS) {
  return PAGED ? ov + (size_t)to * (size_t)TS + SLOT_OV : ov + to;
}

template <bool PAGED>
__device__ __forceinline__ void load_tags(const Bases& B, const TileTable& TT, int tile, int a, TagRegs& Tg) {
  if (PAGED) {
    const int2 e = TT.tt[tile - TT.tlo];
    const int ek = __builtin_amdgcn_readfirstlane(e.x), ev = __builtin_amdgcn_readfirstlane(e.y);
    Tg.raw = (ek | ev) < 0;                       // a tile with a raw side is skipped here and handled by raw_rows_attend
    Tg.kto = (u32)max(ek, 0); Tg.vto = (u32)max(ev, 0);
    Tg.kfl = reinterpret_cast<const u32*>(B.kov + (size_t)Tg.kto * (size_t)B.TS + SLOT_FL)[a];
    Tg.vfl = reinterpret_cast<const u32*>(B.vov + (size_t)Tg.vto * (size_t)B.TS + SLOT_FL)[a];
  } else {
    const u32 w = (u32)(tile * T + a);
    Tg.kfl = (u32)__builtin_nontemporal_load(B.kfl + w); Tg.vfl = (u32)__builtin_nontemporal_load(B.vfl + w);
    Tg.kto = (u32)B.kto[(u32)tile]; Tg.vto = (u32)B.vto[(u32)tile];
    Tg.raw = 0;
  }
}

// the tile's sign/mantissa and code bytes (paged mode: the slot index comes with the tags)
template <bool PAGED>
__device__ __forceinline__ void load_tile_payload(const Bases& B, int tile, int lane, const TagRegs& Tg, TileRegs& R) {
  if (PAGED) {
    const uint8_t* ks = B.kov + (size_t)__builtin_amdgcn_readfirstlane(Tg.kto) * (size_t)B.TS;
    const uint8_t* vs = B.vov + (size_t)__builtin_amdgcn_readfirstlane(Tg.vto) * (size_t)B.TS;
    load_payload(ks, ks + SLOT_CD, lane, R.k.pay);
    load_payload(vs, vs + SLOT_CD, lane, R.v.pay);
  } else {
    // uniform 64-bit base + 32-bit byte offset per lane (one add per array; a head's arrays stay below 4 GiB, checked on the host)
    const u32 so = (u32)tile * TILE_SM + 16u * (u32)lane, co = (u32)tile * TILE_CD + 4u * (u32)lane;
    R.k.pay.s0 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B.ksm + so));
    R.k.pay.s1 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B.ksm + so + 1024u));
    R.v.pay.s0 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B.vsm + so));
    R.v.pay.s1 = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(B.vsm + so + 1024u));
    R.k.pay.c0 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.kcd + co));
    R.k.pay.c1 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.kcd + co + 256u));
    R.k.pay.c2 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.kcd + co + 512u));
    R.v.pay.c0 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.vcd + co));
    R.v.pay.c1 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.vcd + co + 256u));
    R.v.pay.c2 = __builtin_nontemporal_load(reinterpret_cast<const u32*>(B.vcd + co + 512u));
  }
}
// the lane's escape position from the tag words, and the 8 escape bytes from there on
template <bool PAGED>
__device__ __forceinline__ void load_tile_escapes(const Bases& B, int lane, const TagRegs& Tg, TileRegs& R) {
  const int q = lane >> 4;
  // escape bytes per line of K (low half) and V (high half): one scan for both
  const u32 rb = (u32)esc_bytes(Tg.kfl) | ((u32)esc_bytes(Tg.vfl) << 16);
  const u32 excl = row_scan16(rb) - rb;
  // What the consumer needs of the tag words and tile offsets is computed here, into registers of the tile: the tag registers are
  // then free for the next tags, and nothing has to be copied out of a register that a load is still writing.
  R.k.f = __builtin_amdgcn_ubfe(Tg.kfl, 8 * q, 8); R.v.f = __builtin_amdgcn_ubfe(Tg.vfl, 8 * q, 8);
  R.k.pos0 = (excl & 0xFFFFu) + (u32)esc_prefix(Tg.kfl, 8 * q);
  R.v.pos0 = (excl >> 16) + (u32)esc_prefix(Tg.vfl, 8 * q);
  if (PAGED) {      // the 8-byte window stays inside the slot: a lane whose escape bytes start in the slot's last 7 bytes takes the slow look-up
    const u32 lim = (u32)(B.TS - SLOT_OV - 8);      // TS >= SLOT_OV + 16 (checked on the host)
    R.k.e = load_u32x2_unaligned(esc_of_tile<PAGED>(B.kov, __builtin_amdgcn_readfirstlane(Tg.kto), B.TS) + min(R.k.pos0, lim));
    R.v.e = load_u32x2_unaligned(esc_of_tile<PAGED>(B.vov, __builtin_amdgcn_readfirstlane(Tg.vto), B.TS) + min(R.v.pos0, lim));
  } else {      // stream base (uniform) + 32-bit offset (tile offset + position in the tile)
    R.k.pos0 += Tg.kto; R.v.pos0 += Tg.vto;
    R.k.e = load_u32x2_unaligned(B.kov + R.k.pos0);
    R.v.e = load_u32x2_unaligned(B.vov + R.v.pos0);
  }
}
template <bool PAGED>
__device__ __forceinline__ void load_tile(const Bases& B, int tile, int lane, const TagRegs& Tg, TileRegs& R) {
  load_tile_payload<PAGED>(B, tile, lane, Tg, R);
  load_tile_escapes<PAGED>(B, lane, Tg, R);
}

// ---------------------------------------------------------------------------------------------------- one tile pair
struct WaveState { f32x4 acc[8]; float m_run, mu_run, l_run; };     // acc[i][r] = O[head a][group 4q+r, element i]; m in raw score units

// unit decode with the escape contribution already expanded to exponent-field words x (see AttnLds::xlut)
__device__ __forceinline__ void decode_unit_x(u32 slo, u32 shi, u32 g24, const u32x4& x, const u32x4& bw, u32* __restrict__ out) {
  // low-half codes stay at bits 3p, high-half codes move to bits 16 + 3p; the bits this leaves at 12..15 and 28..31 never reach the
  // fields the four masks below keep
  const u32 cw = ((g24 << 4) & 0x0FFF0000u) | (g24 & ~0x0FFF0000u);
  const u32 c0 = (cw << 7) & 0x03800380u, c1 = (cw << 4) & 0x03800380u, c2 = (cw << 1) & 0x03800380u, c3 = (cw >> 2) & 0x03800380u;
  // bw: the base words of the unit's tier (3-bit base, or 4-bit base for promoted and raw groups: their x holds hi5 - base4)
  const u32 e0 = c0 + bw[0] + x[0], e1 = c1 + bw[1] + x[1], e2 = c2 + bw[2] + x[2], e3 = c3 + bw[3] + x[3];
  out[0] = (e0 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x04040000u) & ~EXP_MASK2);
  out[1] = (e1 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x05050101u) & ~EXP_MASK2);
  out[2] = (e2 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x06060202u) & ~EXP_MASK2);
  out[3] = (e3 & EXP_MASK2) | (__builtin_amdgcn_perm(shi, slo, 0x07070303u) & ~EXP_MASK2);
}
// raw group: 8 x 5 high exponent bits (40-bit little endian in lo/hi) as exponent-field words MINUS the 4-bit base words,
// so that code + base4 + x reproduces code | hi5 << 3 exactly (32-bit arithmetic, the base cancels)
__device__ __forceinline__ u32x4 raw_x_words(u32 lo, u32 hi, const u32x4& b4w) {
  u32x4 x;
  x[0] = (((lo) & 31u) << 10 | ((lo >> 20) & 31u) << 26) - b4w[0];
  x[1] = (((lo >> 5) & 31u) << 10 | ((lo >> 25) & 31u) << 26) - b4w[1];
  x[2] = (((lo >> 10) & 31u) << 10 | (__builtin_amdgcn_alignbit(hi, lo, 30) & 31u) << 26) - b4w[2];
  x[3] = (((lo >> 15) & 31u) << 10 | ((hi >> 3) & 31u) << 26) - b4w[3];
  return x;
}

// The x words of the lane's four units.  Common case: 4-bit groups only -> one v_perm + four table reads.  A wave with a raw
// group somewhere (most tiles, few lanes) patches those units from the prefetched bytes.  A lane with two or more raw groups
// (its bytes may not fit the 8 prefetched ones) re-reads memory: only the SLOW instantiation contains those loads, so the
// common instantiation has no memory access between the prefetch and the products.
// bw[u]: the exponent-base words of unit u's tier, read from the block's LDS table: one table row per (tier, group), so the tier
// select costs an address bit instead of four conditional moves per unit.
// lim (SLOW only): last offset from esc_tile at which an 8-byte load may start (paged pool: the slot's end - 8; a stream: no limit).
template <int KIND, bool SLOW>
__device__ __forceinline__ void unit_x_words(const KindRegs& R, const AttnLds& L, const uint8_t* __restrict__ esc_tile, u32 lim, int a, int q,
                                             u32x4* __restrict__ x, u32x4* __restrict__ bw) {
  const u32 tag8 = R.f;
  const u32 eb4 = __builtin_amdgcn_perm(R.e[1], R.e[0], L.sel[tag8]);
  const u32x4* tab = KIND == KIND_K ? &L.bwk[0][4 * q] : &L.bwv[0][a];      // row of unit 0 at tier 0; tier 1 is NG rows further
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    x[u] = L.xlut[(eb4 >> (8 * u)) & 0xFFu];
    bw[u] = tab[(KIND == KIND_K ? u : 0) + NG * ((tag8 >> (2 * u)) & 1u)];
  }
  if (__builtin_amdgcn_ballot_w64((tag8 & 0xAAu) != 0u || (SLOW && R.pos0 > lim))) {
    const u64 e64 = (u64)R.e[0] | ((u64)R.e[1] << 32);
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      if (((tag8 >> (2 * u)) & 3u) == 3u) {          // offset = number of 4-bit groups below (a raw one below is handled next)
        const u64 v = e64 >> (8 * __popc(tag8 & (0x55u & ((1u << (2 * u)) - 1u))));
        x[u] = raw_x_words((u32)v, (u32)(v >> 32), bw[u]);
      }
    }
    if (SLOW && (__popc(tag8 & 0xAAu) >= 2 || R.pos0 > lim)) {
      u32 off = 0u;
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const u32 t = (tag8 >> (2 * u)) & 3u;
        if (t) {
          const u32 at = R.pos0 + off, from = min(at, lim);      // bytes past the limit are not this unit's: load lower, shift down
          const u64 v = load_u64_unaligned(esc_tile + from) >> (8u * (at - from));
          // The loaded bytes are waited for here, in the block that issues the load: their two users below sit in separate divergent
          // blocks, and a load that is still pending on the path past both makes the compiler wait for every load in flight wherever
          // its register is reused, on the common path as well.
          u32 vlo = (u32)v, vhi = (u32)(v >> 32);
          asm volatile("" : "+v"(vlo), "+v"(vhi));
          x[u] = t == 1u ? L.xlut[vlo & 0xFFu] : raw_x_words(vlo, vhi, bw[u]);
        }
        off += (u32)tag_size(t);
      }
    }
  }
}

// PARTIAL: the tile is the last one of the sequence and only partly filled (rows >= S are masked out).  It is a template
// parameter, not a run-time branch, so that no branch separates the score MFMAs from the first read of their result.
template <bool PAGED, bool PARTIAL>
__device__ __forceinline__ void consume(const TileRegs& R, WaveState& st, const AttnLds& L, const Bases& B,
                                        u32 kto, u32 vto, int tile, int S, float scale_log2e, int a, int q,
                                        const u32x4 (&qf)[4]) {
  // A tile needs the SLOW look-up of its escape words when some lane holds two or more raw groups (about 1 tile in 100 at 0.3 % raw
  // groups).  The choice is one wave-uniform branch around the look-ups only, ahead of all the matrix products of the tile.
  u32x4 xk[4], xv[4], bk[4], bv[4];
  const u32 kr = R.k.f & 0xAAu, vr = R.v.f & 0xAAu;
  const u32 lim = PAGED ? (u32)(B.TS - SLOT_OV - 8) : 0xFFFFFFFFu;      // paged pool: the 8 prefetched bytes were taken from no further than this
  bool slow = ((kr & (kr - 1u)) | (vr & (vr - 1u))) != 0u;
  if (PAGED) slow |= max(R.k.pos0, R.v.pos0) > lim;      // (also lanes without escape bytes: a position that far into a slot is rare)
  const bool any_slow = __builtin_amdgcn_ballot_w64(slow) != 0;
  if (__builtin_expect(any_slow, 0)) {
    unit_x_words<KIND_K, true>(R.k, L, PAGED ? esc_of_tile<PAGED>(B.kov, kto, B.TS) : B.kov, lim, a, q, xk, bk);
    if (!WAVES12) unit_x_words<KIND_V, true>(R.v, L, PAGED ? esc_of_tile<PAGED>(B.vov, vto, B.TS) : B.vov, lim, a, q, xv, bv);
  } else {
    unit_x_words<KIND_K, false>(R.k, L, nullptr, lim, a, q, xk, bk);
    if (!WAVES12) unit_x_words<KIND_V, false>(R.v, L, nullptr, lim, a, q, xv, bv);
  }
  // ---- scores: S[tok 4q+r][head a]
  f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi, w[4];
    unit_sm(R.k.pay, u, slo, shi);
    decode_unit_x(slo, shi, unit_code_word(R.k.pay.c0, R.k.pay.c1, R.k.pay.c2, u), xk[u], bk[u], w);
    const u32x4 av = {w[0], w[1], w[2], w[3]};
    const u32x4 qu = WAVES12 ? L.qw[a][4 * q + u] : qf[u];
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av), __builtin_bit_cast(bf16x8, qu), sacc, 0, 0, 0);
  }
  if (WAVES12) {      // measurement build: the V side's look-ups only now, when the K side's registers are free
    if (__builtin_expect(any_slow, 0)) unit_x_words<KIND_V, true>(R.v, L, PAGED ? esc_of_tile<PAGED>(B.vov, vto, B.TS) : B.vov, lim, a, q, xv, bv);
    else unit_x_words<KIND_V, false>(R.v, L, nullptr, lim, a, q, xv, bv);
  }
  // ---- online softmax per head a over the tile's 16 tokens (4 in this lane, 4 quads); exp2(score * scale*log2e - mu)
  const int tok0 = tile * T + 4 * q;
  if (PARTIAL) {
#pragma unroll
    for (int r = 0; r < 4; ++r) sacc[r] = tok0 + r >= S ? -INFINITY : sacc[r];
  }
  const float tmax = quad_rows_max(fmaxf(fmaxf(sacc[0], sacc[1]), fmaxf(sacc[2], sacc[3])));
  if (__builtin_amdgcn_ballot_w64(tmax > st.m_run)) {             // the running maximum of some head grows (rare after the first tiles)
    const float mn = fmaxf(st.m_run, tmax), mu = mn == -INFINITY ? 0.f : mn * scale_log2e;
    const float alpha = __builtin_amdgcn_exp2f(st.m_run == -INFINITY ? -INFINITY : st.mu_run - mu);
    st.l_run *= alpha;
#pragma unroll
    for (int i = 0; i < 8; ++i) st.acc[i] *= alpha;
    st.m_run = mn; st.mu_run = mu;
  }
  float p[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], scale_log2e, -st.mu_run));
  st.l_run += (p[0] + p[1]) + (p[2] + p[3]);
  const u32x2 pw = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3])};
  const s16x4 pb = __builtin_bit_cast(s16x4, pw);
  // ---- values: decode the lane's 4 tokens of group a, regroup as token pairs per element, accumulate O^T
  u32 W[4][4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    u32 slo, shi;
    unit_sm(R.v.pay, u, slo, shi);
    decode_unit_x(slo, shi, unit_code_word(R.v.pay.c0, R.v.pay.c1, R.v.pay.c2, u), xv[u], bv[u], W[u]);
  }
  if (PARTIAL) {                // rows beyond the sequence must not reach the product
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int pp = 0; pp < 4; ++pp) W[u][pp] = tok0 + u >= S ? 0u : W[u][pp];
  }
#pragma unroll
  for (int pp = 0; pp < 4; ++pp) {
    const u32x2 lo = {__builtin_amdgcn_perm(W[1][pp], W[0][pp], 0x05040100u), __builtin_amdgcn_perm(W[3][pp], W[2][pp], 0x05040100u)};
    const u32x2 hi = {__builtin_amdgcn_perm(W[1][pp], W[0][pp], 0x07060302u), __builtin_amdgcn_perm(W[3][pp], W[2][pp], 0x07060302u)};
    st.acc[pp] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, lo), pb, st.acc[pp], 0, 0, 0);
    st.acc[pp + 4] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, hi), pb, st.acc[pp + 4], 0, 0, 0);
  }
}

// Next tile for a wave from the block's counter in LDS (lane 0's value counts).  The caller makes it uniform only when it needs it,
// one tile later, so that no wave waits for the LDS atomic.  Indices past the block's range come back as NO_TILE.
constexpr int NO_TILE = 0x3FFFFFFF;
__device__ __forceinline__ int take_tile(int* ctr, int hi, int lane) {
  int v = 0;
  if (lane == 0) { v = atomicAdd(ctr, 1); v = v < hi ? v : NO_TILE; }
  return v;
}
__device__ __forceinline__ int uniform_tile(int v) { return __builtin_amdgcn_readfirstlane(v); }

// ---------------------------------------------------------------------------------------------------- main kernel
// NW = waves per block: 4 (two blocks per CU) or 8 (one block per CU: half as many partials to merge for the same occupancy)
// HOST_LEN: the compressed length of every addressed head is the kernel argument S_all (not read from memory)
template <bool PAGED, int NW, bool HOST_LEN>
__global__ void __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) k_attn_split(const AttnArgs A) {
  constexpr int NT = 64 * NW;
  // one LDS object so that the tables the tile loop reads sit at the lowest addresses (immediate offsets of the LDS loads)
  struct BlockLds { AttnLds L; int next_tile; int2 tile_table[PAGED ? MAX_CHUNK : 1]; MergeLds<NW> M; };
  __shared__ BlockLds lds;
  AttnLds& L = lds.L; MergeLds<NW>& M = lds.M; int2* tile_table = lds.tile_table; int& next_tile = lds.next_tile;
  const int tid = threadIdx.x;
  GAAC_STAMP(0);
  // One-dimensional grid, numbered split-fastest: the splits of one kv head go round the eight XCDs (workgroups are dealt to XCDs in
  // turn) instead of all landing on one, so heads with heavier tiles load every XCD alike.
  // The start of a block is a chain of dependent loads (arguments -> slot -> lengths and stream starts -> tag words -> escape bytes),
  // each a trip to memory with nothing else to do: issue everything a level allows before the first use of any of its results.
  // Level 0: the kernel arguments, forced into scalar registers together (otherwise each is fetched where it is first used).
  if (PAGED)
    asm volatile("" ::"s"(A.q), "s"(A.sl), "s"(A.bt), "s"(A.mt), "s"(A.pool), "s"(A.raw), "s"(A.k.base3), "s"(A.k.base4), "s"(A.v.base3),
                 "s"(A.v.base4), "s"(A.nsplit), "s"(A.n_kv), "s"(A.n_q), "s"(A.G), "s"(A.NB), "s"(A.bt_stride), "s"(A.TS));
  else
    asm volatile("" ::"s"(A.q), "s"(A.slot), "s"(A.sl), "s"(A.k.sm), "s"(A.k.cd), "s"(A.k.flags), "s"(A.k.tile_off), "s"(A.k.ovf),
                 "s"(A.k.head_start), "s"(A.k.base3), "s"(A.k.base4), "s"(A.v.sm), "s"(A.v.cd), "s"(A.v.flags), "s"(A.v.tile_off),
                 "s"(A.v.ovf), "s"(A.v.head_start), "s"(A.v.base3), "s"(A.v.base4), "s"(A.kt), "s"(A.tl), "s"(A.nsplit), "s"(A.n_kv),
                 "s"(A.n_q), "s"(A.G), "s"(A.NB), "s"(A.S_pad), "s"(A.tcap));
  // Paged pool: the launch can take the place of gaac_paged_free (it pops nothing, so pushes are safe here): the grid's last block, the
  // one with the least to do, pushes the queued raw tiles back before its own work.  The wait keeps the stores' bookkeeping out of
  // the code every block runs.
  if (PAGED && A.freeq != nullptr && blockIdx.x == gridDim.x - 1) {
    for (int i = tid; i < A.n_free; i += NT) { const int r = A.freeq[i]; if (r >= 0) A.stack[atomicAdd(A.top, 1)] = r; }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  }
  // Paged pool: the split index is rotated by the head index: the last split of a sequence carries the raw tile that is still filling,
  // and with equal split counts all of them would otherwise sit on the same XCD, which then finishes long after the others.
  const int bh = (int)blockIdx.x / A.nsplit, split = ((int)blockIdx.x + (PAGED ? bh : 0)) % A.nsplit;
  int b = bh / A.n_kv, S_ranked = -1;
  const int kvh = bh % A.n_kv, G = A.G;
  if (PAGED) {
    // Ragged batches: blocks start in index order, so the longest sequences go first and the short ones fill the end of the launch
    // (in batch order a long sequence that happens to come last runs on with most of the GPU idle).  Batch row = the sequence whose
    // length has rank b; every block ranks the lengths itself (thread i counts the sequences ahead of sequence i).
    const int Bn = (int)gridDim.x / (A.nsplit * A.n_kv);
    if (Bn > 1 && Bn <= NT) {
      int* lens = reinterpret_cast<int*>(&M.acc[0][0][0]);      // the merge buffer is idle until the tile loop has ended
      const int mine = tid < Bn ? max(A.sl[tid], 0) : 0;
      if (tid < Bn) lens[tid] = mine;
      __syncthreads();
      if (tid < Bn) {
        int rank = 0;
        for (int j = 0; j < Bn; ++j) { const int lj = lens[j]; rank += (lj > mine || (lj == mine && j < tid)) ? 1 : 0; }
        if (rank == b) { lens[NT] = tid; lens[NT + 1] = mine; }
      }
      __syncthreads();
      b = __builtin_amdgcn_readfirstlane(lens[NT]); S_ranked = __builtin_amdgcn_readfirstlane(lens[NT + 1]);
    }
  }
  const long qh0 = (long)b * A.n_q + (long)kvh * G;
  // Level 1: the slot of the batch row; the query rows do not depend on it
  TableRegs Tr;
  if (tid < 256) tables_load_q(Tr, tid, A.q + qh0 * D, G);
  // (no slot map = row b attends over cache heads b*n_kv ..: one level of dependent loads less)
  const int slot = PAGED ? 0 : (A.slot ? A.slot[b] : b), ch = PAGED ? kvh : (slot < 0 ? 0 : slot) * A.n_kv + kvh;
  // Level 2: everything indexed by the cache head
  int S, TLh = 0; long khs = 0, vhs = 0;
  if (PAGED) S = S_ranked >= 0 ? S_ranked : max(A.sl[b], 0);
  else {
    // lengths known to the host (a Page) come as a kernel argument: the tile range, and with it the first payload loads, then depend on
    // nothing but the arguments
    // These values are needed late (escape bytes, tail).  The index goes through a vector register the compiler knows nothing
    // about, so that the loaded values stay in vector registers until readfirstlane fetches them where they are used; a value the
    // compiler knows to be uniform is moved to a scalar register, and waited for, right where it is loaded.
    int chv = ch;
    asm volatile("" : "+v"(chv));
    khs = A.k.head_start[chv]; vhs = A.v.head_start[chv];
    TLh = (A.kt ? A.tl : A.k.head_start)[chv];      // no branch between the loads of this level
    if (HOST_LEN) S = A.S_all;
    else S = A.sl[ch];
    if (slot < 0) S = 0;
  }
  if (tid < 256) tables_load_bases(Tr, tid, A.k.base3, A.k.base4, A.v.base3, A.v.base4, ch % A.NB);

  const int ntiles = (S + T - 1) / T, chunk = (ntiles + A.nsplit - 1) / A.nsplit;
  const int tlo = min(split * chunk, ntiles), thi = min(tlo + chunk, ntiles);
  const int thi_fast = PAGED ? min(thi, tlo + MAX_CHUNK) : thi;      // the pipelined loop's range: what one fill of the LDS tile table covers
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, a = lane & 15, q = lane >> 4;
  Bases B;
  TileTable TT{tile_table, tlo};
  if (PAGED) {
    // logical tile -> block table -> mode table (paged_kernel.py:137-138), resolved once per block into LDS
    B.kov = B.vov = A.pool; B.TS = A.TS;
    B.ksm = B.kcd = B.vsm = B.vcd = nullptr; B.kfl = B.kto = B.vfl = B.vto = nullptr;
    for (int i = tid; i < thi_fast - tlo; i += NT) {
      const long pc = (long)A.bt[(long)b * A.bt_stride + tlo + i] * (2 * A.n_kv) + 2 * kvh;
      tile_table[i] = int2{A.mt[pc], A.mt[pc + 1]};
    }
    __syncthreads();
  } else {
    const long rowb = (long)ch * A.S_pad, tileb = (long)ch * (A.S_pad / T);
    // (the escape streams start at head_start[ch], a loaded value: they are set where the first escape bytes are fetched, so that the
    // loads issued until then do not wait for it)
    B.ksm = A.k.sm + rowb * D; B.kcd = A.k.cd + rowb * CB; B.kfl = A.k.flags + rowb; B.kto = A.k.tile_off + tileb; B.kov = nullptr;
    B.vsm = A.v.sm + rowb * D; B.vcd = A.v.cd + rowb * CB; B.vfl = A.v.flags + rowb; B.vto = A.v.tile_off + tileb; B.vov = nullptr;
    B.TS = 0;
  }

  // Tiles are handed out dynamically: each wave starts with tiles tlo + wave and tlo + NW + wave and takes every further one from
  // a counter in LDS.  Of the two waves that share a SIMD the older one wins the issue arbitration and runs ahead; with a static
  // split it would finish long before the other, which then runs alone and cannot hide its own latencies.  Ping-pong registers
  // R0/R1; tag words are fetched one tile further ahead; indices past the end are clamped for the loads (no load sits under a
  // branch the consumer has to join) and not consumed.  A partly filled last tile of the sequence is handled at the end by wave 0.
  // logical tile index i of this block -> tile tlo + i
  const int full = ntiles - ((S % T) != 0 ? 1 : 0);      // tiles with all 16 rows
  const int n_own = max(min(thi_fast, full) - tlo, 0);
  const int icl = max(n_own - 1, 0);
#define TILE(i) (tlo + (i))
  int iA = wave, iB = wave + NW;
  TileRegs R0, R1;
  // Two sets of tag registers, used in turn: a set is loaded one tile before the payload that needs it, read where that payload's
  // escape bytes are fetched, and then free.  (Paged pool: slot indices and the raw mark of the tile in R0 / R1, scalar values.)
  TagRegs Tg, TgB;
  struct TileMeta { u32 kto, vto; int raw; } m0 = {0u, 0u, 0}, m1 = {0u, 0u, 0};
  const bool any_tile = iA < n_own;
  // The wave's first tile: tag words and payload.  Without a branch where the addresses are always valid (a wave without tiles reads
  // a tile it does not consume): behind a branch the compiler can no longer count the loads in flight and turns every later wait
  // into a wait for all of them.  The escape bytes, which need the tag words and the stream start, follow after the block tables.
  if (!PAGED || any_tile) {
    const int tA = min(TILE(min(iA, icl)), max(ntiles - 1, 0));
    load_tags<PAGED>(B, TT, tA, a, Tg);
    load_tile_payload<PAGED>(B, tA, lane, Tg, R0);
  }
  if (tid == 0) next_tile = 2 * NW;
  // this launch's epoch of the fused merge: one more load of the start-up batch, its value is needed when the block is done
  const u32 epoch = load_epoch(A, bh);
  GAAC_STAMP(6);
  if (tid < 256) tables_store(L, Tr, tid, G);
  GAAC_STAMP(7);
  if (tid < GMAX) { M.m[NW][tid] = -INFINITY; M.l[NW][tid] = 0.f; }
  lds_barrier();        // block tables are ready (a barrier that does not wait for the tile loads in flight)
  GAAC_STAMP(1);
  // Q as the B operand of the score product: lane (head a, quad q), product u covers group 4q+u in word order (e, e+4);
  // exponent-base words of the lane's units
  u32x4 qf[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) qf[u] = L.qw[a][4 * q + u];

  WaveState st;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m_run = -INFINITY; st.mu_run = 0.f; st.l_run = 0.f;

  // ---- the raw tail of the cache head: wave 0 of the last split's block, before it joins the tile hand-out
  if (!PAGED && A.kt && split == A.nsplit - 1 && wave == 0) {
    const int TL = slot < 0 ? 0 : min(__builtin_amdgcn_readfirstlane(TLh), A.tcap);
    if (TL > 0) {
      // probabilities go through this wave's own merge slot: the other waves write theirs as soon as they run out of tiles
      float (*sc)[T] = reinterpret_cast<float (*)[T]>(&M.acc[0][0][0]);
      wave_rows_attend(sc, A.kt + (long)ch * A.tcap * D, A.vt + (long)ch * A.tcap * D, TL, A.q + qh0 * D, A.scale_log2e, G, lane,
                       M.m[NW], M.l[NW], M.acc[NW]);
    }
  }

  if (!PAGED) { B.kov = A.k.ovf + __builtin_amdgcn_readfirstlane((int)khs); B.vov = A.v.ovf + __builtin_amdgcn_readfirstlane((int)vhs); }
  if (any_tile) {
    if (PAGED) m0 = TileMeta{Tg.kto, Tg.vto, Tg.raw};
    load_tile_escapes<PAGED>(B, lane, Tg, R0);
    load_tags<PAGED>(B, TT, TILE(min(iB, icl)), a, TgB);
    int vC = take_tile(&next_tile, n_own, lane);
    // The loop is entered with the loads in flight in the same order as on its back edge (tile, then the next tile's tags), so the
    // waits inside it stay waits for exactly the loads they need.
    while (true) {        // R0 = tile iA, TgB = tags of tile iB
      if (PAGED) m1 = TileMeta{TgB.kto, TgB.vto, TgB.raw};
      load_tile<PAGED>(B, TILE(min(iB, icl)), lane, TgB, R1);
      const int vD = take_tile(&next_tile, n_own, lane);
      const int iC = uniform_tile(vC);
      load_tags<PAGED>(B, TT, TILE(min(iC, icl)), a, Tg);
      if (!PAGED || !m0.raw) consume<PAGED, false>(R0, st, L, B, m0.kto, m0.vto, TILE(iA), S, A.scale_log2e, a, q, qf);
      if (iB >= n_own) break;
      if (PAGED) m0 = TileMeta{Tg.kto, Tg.vto, Tg.raw};
      load_tile<PAGED>(B, TILE(min(iC, icl)), lane, Tg, R0);
      const int vE = take_tile(&next_tile, n_own, lane);
      const int iD = uniform_tile(vD);
      load_tags<PAGED>(B, TT, TILE(min(iD, icl)), a, TgB);
      if (!PAGED || !m1.raw) consume<PAGED, false>(R1, st, L, B, m1.kto, m1.vto, TILE(iB), S, A.scale_log2e, a, q, qf);
      if (iC >= n_own) break;
      iA = iC; iB = iD; vC = vE;
    }
  }
#undef TILE
  // arrival mark of the block for the fused merge (see merge_heads): the wave has no load in flight here
  if (A.epochs != nullptr && A.nslot > 1 && tid == 0) mark_arrival(A, epoch);
  GAAC_STAMP(2);
#ifdef GAAC_PHASE_TIMING
  if (A.dbg && lane == 0) A.dbg[((long)gridDim.x + blockIdx.x) * 8 + wave] = wall_clock64();
#endif
  // ---- what the pipelined loop left: (1) the partly filled last tile of the sequence; (2) paged pool: a split longer than the LDS tile
  // table goes on in further rounds of MAX_CHUNK tiles (table refilled); (3) paged pool: tiles whose K or V side is a raw tile (the
  // block that is still filling, or escapes that did not fit the slot), attended by the whole block round by round, while the table
  // holds their entries.  Tiles of (1) and (2) are taken by the waves in turn, one at a time without the prefetch pipeline (of the
  // block's waves some compute while others wait for their tile; both cases are rare), through ONE instantiation of the masking tile
  // code.
  if (tlo < thi) {
    bool raw_started = false;
    for (int c0 = tlo;;) {
      const int c1 = PAGED ? min(c0 + MAX_CHUNK, thi) : thi;
      if (PAGED && c0 != tlo) {
        __syncthreads();      // everybody is done with the previous round's entries
        for (int i = tid; i < c1 - c0; i += NT) {
          const long pc = (long)A.bt[(long)b * A.bt_stride + c0 + i] * (2 * A.n_kv) + 2 * kvh;
          tile_table[i] = int2{A.mt[pc], A.mt[pc + 1]};
        }
        __syncthreads();
        TT.tlo = c0;
      }
      for (int t = (c0 == tlo ? tlo + n_own : c0) + wave; t < c1; t += NW) {      // first round: only the partial tile is left (wave 0)
        load_tags<PAGED>(B, TT, t, a, Tg);
        load_tile<PAGED>(B, t, lane, Tg, R0);
        if (!PAGED || !Tg.raw) consume<PAGED, true>(R0, st, L, B, Tg.kto, Tg.vto, t, S, A.scale_log2e, a, q, qf);
      }
      if (PAGED) {
        bool mine = false;
        for (int i = tid; i < c1 - c0; i += NT) mine |= (tile_table[i].x | tile_table[i].y) < 0;
        if (__syncthreads_or(mine)) {
          RawScratch& R = *reinterpret_cast<RawScratch*>(&M.acc[0][0][0]);
          if (!raw_started) {
            for (int g = tid >> 7; g < G; g += NT / 128) M.acc[NW][g][tid & 127] = 0.f;
            raw_rows_begin<NT>(R, A, qh0, G, tid);
            raw_started = true;
          }
          const uint8_t* b3k = A.k.base3 + (long)(ch % A.NB) * D; const uint8_t* b4k = A.k.base4 + (long)(ch % A.NB) * D;
          const uint8_t* b3v = A.v.base3 + (long)(ch % A.NB) * D; const uint8_t* b4v = A.v.base4 + (long)(ch % A.NB) * D;
          for (int i = 0; i < c1 - c0; ++i) {
            const int2 e = tile_table[i];
            if ((e.x | e.y) >= 0) continue;
            const u16* krows = R.krows; const u16* vrows = R.vrows;
            if (e.x < 0) krows = A.raw + (long)(~e.x) * T * D;
            else if (wave == 0) {
              const uint8_t* sl = A.pool + (size_t)e.x * (size_t)A.TS;
              decode_tile_rows<KIND_K>(sl, sl + SLOT_CD, reinterpret_cast<const int*>(sl + SLOT_FL), sl + SLOT_OV, b3k, b4k, lane, T, R.krows, D);
            }
            if (e.y < 0) vrows = A.raw + (long)(~e.y) * T * D;
            else if (wave == 1) {
              const uint8_t* sl = A.pool + (size_t)e.y * (size_t)A.TS;
              decode_tile_rows<KIND_V>(sl, sl + SLOT_CD, reinterpret_cast<const int*>(sl + SLOT_FL), sl + SLOT_OV, b3v, b4v, lane, T, R.vrows, D);
            }
            raw_rows_attend<NT>(R, krows, vrows, min(T, S - (c0 + i) * T), A.scale_log2e, G, tid, M.m[NW], M.l[NW], M.acc[NW]);
            __syncthreads();      // staging rows are free again
          }
        }
      }
      c0 = c1;
      if (c0 >= thi) break;
    }
  }
  // The accumulators are MFMA results: keep their first non-MFMA read a full MFMA latency away on every path.
  asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
  GAAC_STAMP(3);
  float l_run = quad_rows_sum(st.l_run);
  const float m_run = st.m_run == -INFINITY ? -INFINITY : st.mu_run;     // partial maxima are stored in the base-2 domain
  f32x4 (&acc)[8] = st.acc;

  // ---- merge the waves of the block, write the split's partial
  if (a < G) {
    if (q == 0) { M.m[wave][a] = m_run; M.l[wave][a] = l_run; }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) M.acc[wave][a][chan_v(8 * (4 * q + r) + i)] = acc[i][r];
  }
  GAAC_MSTAMP(5, wall_clock64());
  lds_barrier();      // only LDS data crosses (a full barrier would also wait for the acknowledgement of the arrival mark)
  GAAC_MSTAMP(6, wall_clock64());
  const bool fused = A.epochs != nullptr;
  const int mergers = merge_ranks(G, A.nslot), rank = (int)blockIdx.x % A.nsplit - (A.nsplit - mergers);      // the head's last blocks to start
  const int d = tid & 127;
  for (int g = tid >> 7; g < G; g += NT / 128) {
    // every LDS read up front and none under a branch: nine dependent round trips otherwise
    float mv[NW + 1], lv[NW + 1], av[NW + 1];
#pragma unroll
    for (int w = 0; w < NW + 1; ++w) { mv[w] = M.m[w][g]; lv[w] = M.l[w][g]; av[w] = M.acc[w][g][d]; }
    float Mx = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW + 1; ++w) Mx = fmaxf(Mx, mv[w]);
    float Lc = 0.f, Ac = 0.f;
#pragma unroll
    for (int w = 0; w < NW + 1; ++w) {
      const bool live = mv[w] != -INFINITY;          // an empty partial's accumulator may hold anything
      const float f = live ? __builtin_amdgcn_exp2f(mv[w] - Mx) : 0.f;
      Lc += lv[w] * f; Ac += (live ? av[w] : 0.f) * f;
    }
    const long pidx = (qh0 + g) * A.nslot + split;
    if (!fused) {
      if (d == 0) { store_partial(A.pm + pidx, Mx); store_partial(A.pl + pidx, Lc); }
      store_partial(A.pa + pidx * D + d, Ac);
    } else if (A.nslot == 1) {      // the only partial of its rows: it is the result
      A.out[(qh0 + g) * D + d] = __builtin_bit_cast(u16, (__bf16)(Lc > 0.f ? Ac / Lc : 0.f));
    } else {
      if (d == 0) { ll_store(reinterpret_cast<u64*>(A.pm) + pidx, Mx, epoch); ll_store(reinterpret_cast<u64*>(A.pl) + pidx, Lc, epoch); }
      ll_store(reinterpret_cast<u64*>(A.pa) + pidx * D + d, Ac, epoch);
    }
  }
  GAAC_STAMP(4);
  if (fused && rank >= 0 && A.nslot > 1) {
    lds_barrier();      // every thread is done with the block-merge buffer, which becomes the mergers' scratch
    merge_heads<NW>(A, qh0, G, epoch, rank, mergers, tid, *reinterpret_cast<MergeScratch<(NW > 8 ? 8 : NW)>*>(&M.acc[0][0][0]));
  }
  GAAC_STAMP(5);
}

// ---------------------------------------------------------------------------------------------------- split merge
__global__ void __launch_bounds__(512) k_attn_combine(const float* __restrict__ pm, const float* __restrict__ pl, const float* __restrict__ pa,
                                                      u16* __restrict__ out, int nslot) {
  __shared__ float fs[MAX_SLOTS];
  __shared__ float red[8];
  __shared__ float part[3][D];
  const int qh = blockIdx.x, tid = threadIdx.x, wv = tid >> 6;
  float m = -INFINITY;
  for (int s = tid; s < nslot; s += 512) m = fmaxf(m, pm[(long)qh * nslot + s]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o, 64));
  if ((tid & 63) == 0) red[wv] = m;
  __syncthreads();
  float M = red[0];
#pragma unroll
  for (int w = 1; w < 8; ++w) M = fmaxf(M, red[w]);
  __syncthreads();
  float l = 0.f;
  for (int s = tid; s < nslot; s += 512) {
    const float v = pm[(long)qh * nslot + s];
    const float f = v == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(v - M);
    fs[s] = f; l += pl[(long)qh * nslot + s] * f;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) l += __shfl_xor(l, o, 64);
  if ((tid & 63) == 0) red[wv] = l;
  __syncthreads();
  float Lsum = 0.f;
#pragma unroll
  for (int w = 0; w < 8; ++w) Lsum += red[w];
  const int d = tid & 127, part_id = tid >> 7;      // four slot-interleaved partial sums per output element
  float acc = 0.f;
#pragma unroll 4
  for (int s = part_id; s < nslot; s += 4) acc += pa[((long)qh * nslot + s) * D + d] * fs[s];
  if (part_id) part[part_id - 1][d] = acc;
  __syncthreads();
  if (part_id == 0) {
    acc += part[0][d] + part[1][d] + part[2][d];
    const float o = Lsum > 0.f ? acc / Lsum : 0.f;
    out[(long)qh * D + d] = __builtin_bit_cast(u16, (__bf16)o);
  }
}

// ---------------------------------------------------------------------------------------------------- uncompressed baseline
// Decode attention over plain BF16 K/V [cache head][token][128] with the same structure as k_attn_split (same split / wave / MFMA
// mapping, online softmax, block merge and fused last-block merge) minus the decoder: the baseline the compressed path is compared
// with on the same GPU.  Args reuse AttnArgs: kt / vt = K / V, S_pad = token stride of a head, tcap = tokens per head.
struct RawTile { u32x4 k[4], v[4]; };
// K: lane (token a, quad q) holds channels 32 j + 8 q .. + 8 for product j.  V: lane (a, q) holds channels 8 a .. 8 a + 8 of tokens 4 q + r.
__device__ __forceinline__ void load_raw_tile(const u16* __restrict__ kh, const u16* __restrict__ vh, int tile, int S, int a, int q, RawTile& R) {
  const int kt = min(tile * T + a, S - 1);
#pragma unroll
  for (int j = 0; j < 4; ++j) R.k[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(kh + (long)kt * D + 32 * j + 8 * q));
#pragma unroll
  for (int r = 0; r < 4; ++r) R.v[r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(vh + (long)min(tile * T + 4 * q + r, S - 1) * D + 8 * a));
}
template <bool PARTIAL>
__device__ __forceinline__ void consume_raw_tile(const RawTile& R, WaveState& st, int tile, int S, float scale_log2e, int q, const u32x4 (&qf)[4]) {
  f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < 4; ++j)
    sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, R.k[j]), __builtin_bit_cast(bf16x8, qf[j]), sacc, 0, 0, 0);
  const int tok0 = tile * T + 4 * q;
  if (PARTIAL) {
#pragma unroll
    for (int r = 0; r < 4; ++r) sacc[r] = tok0 + r >= S ? -INFINITY : sacc[r];
  }
  const float tmax = quad_rows_max(fmaxf(fmaxf(sacc[0], sacc[1]), fmaxf(sacc[2], sacc[3])));
  if (__builtin_amdgcn_ballot_w64(tmax > st.m_run)) {
    const float mn = fmaxf(st.m_run, tmax), mu = mn == -INFINITY ? 0.f : mn * scale_log2e;
    const float alpha = __builtin_amdgcn_exp2f(st.m_run == -INFINITY ? -INFINITY : st.mu_run - mu);
    st.l_run *= alpha;
#pragma unroll
    for (int i = 0; i < 8; ++i) st.acc[i] *= alpha;
    st.m_run = mn; st.mu_run = mu;
  }
  float p[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(sacc[r], scale_log2e, -st.mu_run));
  st.l_run += (p[0] + p[1]) + (p[2] + p[3]);
  const u32x2 pw = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3])};
  const s16x4 pb = __builtin_bit_cast(s16x4, pw);
#pragma unroll
  for (int m = 0; m < 4; ++m) {      // word m of a row = channels 8 a + 2 m, + 1
    u32 w[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) w[r] = PARTIAL && tok0 + r >= S ? 0u : R.v[r][m];
    const u32x2 lo = {__builtin_amdgcn_perm(w[1], w[0], 0x05040100u), __builtin_amdgcn_perm(w[3], w[2], 0x05040100u)};
    const u32x2 hi = {__builtin_amdgcn_perm(w[1], w[0], 0x07060302u), __builtin_amdgcn_perm(w[3], w[2], 0x07060302u)};
    st.acc[2 * m] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, lo), pb, st.acc[2 * m], 0, 0, 0);
    st.acc[2 * m + 1] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, hi), pb, st.acc[2 * m + 1], 0, 0, 0);
  }
}

// NW as in k_attn_split: eight-wave blocks (one per CU) for launches of up to 256 blocks, else four-wave blocks (two per CU)
template <int NW> struct Bf16Lds { u32x4 qw[GMAX][NG]; float m[NW][GMAX], l[NW][GMAX]; float acc[NW + 1][GMAX][D]; };      // acc: also the mergers' scratch
template <int NW>
__global__ void __launch_bounds__(64 * NW, NW == 4 ? 2 : 1) k_bf16_attn_split(const AttnArgs A) {
  constexpr int NT = 64 * NW;
  __shared__ Bf16Lds<NW> L;
  const int bh = (int)blockIdx.x / A.nsplit, split = (int)blockIdx.x % A.nsplit, tid = threadIdx.x;      // a head's blocks are consecutive
  const int b = bh / A.n_kv, kvh = bh % A.n_kv, G = A.G;
  const long qh0 = (long)b * A.n_q + (long)kvh * G;
  const int S = A.sl ? min(max(A.sl[b], 0), A.tcap) : A.tcap;      // per-row lengths on the device (decode steps inside a graph) or one length
  const int ntiles = (S + T - 1) / T, chunk = (ntiles + A.nsplit - 1) / A.nsplit;
  const int tlo = min(split * chunk, ntiles), thi = min(tlo + chunk, ntiles);
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, a = lane & 15, q = lane >> 4;
  const u16* kh = A.kt + (long)bh * A.S_pad * D; const u16* vh = A.vt + (long)bh * A.S_pad * D;
  // dynamic tile hand-out as in k_attn_split
  __shared__ int next_tile;
  const bool part_here = (S % T) != 0 && thi == ntiles && thi > tlo;
  const int thd = thi - (part_here ? 1 : 0), tcl = max(thd - 1, tlo);
  int tA = tlo + wave, tB = tA + NW;
  RawTile R0, R1;
  if (tA < thd) load_raw_tile(kh, vh, tA, S, a, q, R0);
  if (tid == 0) next_tile = tlo + 2 * NW;
  const u32 epoch = load_epoch(A, bh);
  // Q as the B operand: lane (head a, quad q), product j covers channels 32 j + 8 q .. + 8 (rows >= G are zero)
  for (int i = tid; i < GMAX * NG; i += NT) {
    const int h = i >> 4, c = i & 15;
    L.qw[h][c] = h < G ? *reinterpret_cast<const u32x4*>(A.q + (qh0 + h) * D + 8 * c) : u32x4{0u, 0u, 0u, 0u};
  }
  __syncthreads();
  u32x4 qf[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) qf[j] = L.qw[a][4 * j + q];
  WaveState st;
#pragma unroll
  for (int i = 0; i < 8; ++i) st.acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
  st.m_run = -INFINITY; st.mu_run = 0.f; st.l_run = 0.f;
  if (tA < thd) {
    while (true) {
      load_raw_tile(kh, vh, min(tB, tcl), S, a, q, R1);
      const int tC = uniform_tile(take_tile(&next_tile, thd, lane));
      consume_raw_tile<false>(R0, st, tA, S, A.scale_log2e, q, qf);
      if (tB >= thd) break;
      load_raw_tile(kh, vh, min(tC, tcl), S, a, q, R0);
      const int tD = uniform_tile(take_tile(&next_tile, thd, lane));
      consume_raw_tile<false>(R1, st, tB, S, A.scale_log2e, q, qf);
      if (tC >= thd) break;
      tA = tC; tB = tD;
    }
  }
  if (A.nslot > 1 && tid == 0) mark_arrival(A, epoch);
  if (part_here && wave == 0) {
    load_raw_tile(kh, vh, ntiles - 1, S, a, q, R0);
    consume_raw_tile<true>(R0, st, ntiles - 1, S, A.scale_log2e, q, qf);
  }
  asm volatile("s_nop 7\n\ts_nop 7" ::: "memory");
  const float l_run = quad_rows_sum(st.l_run);
  const float m_run = st.m_run == -INFINITY ? -INFINITY : st.mu_run;
  if (a < G) {
    if (q == 0) { L.m[wave][a] = m_run; L.l[wave][a] = l_run; }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) L.acc[wave][a][8 * (4 * q + r) + i] = st.acc[i][r];
  }
  lds_barrier();
  const int mergers = merge_ranks(G, A.nslot), rank = split - (A.nsplit - mergers);
  const int d = tid & 127;
  for (int g = tid >> 7; g < G; g += NT / 128) {
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, L.m[w][g]);
    float Lc = 0.f, Ac = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float f = L.m[w][g] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(L.m[w][g] - M);
      Lc += L.l[w][g] * f; Ac += L.acc[w][g][d] * f;
    }
    const long pidx = (qh0 + g) * A.nslot + split;
    if (A.nslot == 1) A.out[(qh0 + g) * D + d] = __builtin_bit_cast(u16, (__bf16)(Lc > 0.f ? Ac / Lc : 0.f));
    else {
      if (d == 0) { ll_store(reinterpret_cast<u64*>(A.pm) + pidx, M, epoch); ll_store(reinterpret_cast<u64*>(A.pl) + pidx, Lc, epoch); }
      ll_store(reinterpret_cast<u64*>(A.pa) + pidx * D + d, Ac, epoch);
    }
  }
  if (rank >= 0 && A.nslot > 1) {
    lds_barrier();
    merge_heads<NW>(A, qh0, G, epoch, rank, mergers, tid, *reinterpret_cast<MergeScratch<NW>*>(&L.acc[0][0][0]));
  }
}

}  // namespace gaac

using namespace gaac;

#ifdef GAAC_PHASE_TIMING
static long long* g_dbg = nullptr;
extern "C" void gaac_set_phase_buffer(long long* p) { g_dbg = p; }
#endif
static int attn_split_impl(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, void* pm, void* pl, void* pa, unsigned int* epoch, void* out, int S_all, void* stream) {
  GAAC_REQUIRE(n_kv > 0 && n_q > 0 && n_q % n_kv == 0 && n_q / n_kv >= 1 && n_q / n_kv <= GMAX, "GQA group size must be 1..%d (n_q=%d, n_kv=%d)", GMAX, n_q, n_kv);
  GAAC_REQUIRE(smk && ck && fk && tok && ovk && ohsk && b3k && b4k && smv && cv && fv && tov && ovv && ohsv && b3v && b4v, "gaac_attn: null store pointer");
  GAAC_REQUIRE(q && (SL || S_all >= 0) && pm && pl && pa, "gaac_attn: null pointer");
  GAAC_REQUIRE(S_all <= S_pad, "gaac_attn: S_all %d exceeds the token stride %d", S_all, S_pad);
  GAAC_REQUIRE(B > 0 && S_pad > 0 && S_pad % T == 0 && NB > 0, "gaac_attn: bad sizes B=%d S_pad=%d NB=%d", B, S_pad, NB);
  const bool has_tail = kt != nullptr;
  GAAC_REQUIRE(!has_tail || (vt && TL && TCAP >= 1 && TCAP <= T), "gaac_attn: tail needs kt, vt, TL and 1 <= TCAP <= %d", T);
  const int nslot = nsplit;
  GAAC_REQUIRE(nsplit >= 1 && nslot <= MAX_SLOTS, "gaac_attn: nsplit must be in 1..%d", MAX_SLOTS);
  GAAC_REQUIRE(S_pad > 0 && S_pad <= (1 << 24), "gaac_attn: at most %d tokens per cache head (32-bit byte offsets inside a head)", 1 << 24);
  AttnArgs A;
  A.k = StoreView{smk, ck, fk, tok, ovk, ohsk, b3k, b4k};
  A.v = StoreView{smv, cv, fv, tov, ovv, ohsv, b3v, b4v};
  A.q = (const u16*)q; A.pm = (float*)pm; A.pl = (float*)pl; A.pa = (float*)pa; A.slot = slot; A.sl = SL; A.S_all = S_all < 0 ? -1 : S_all;
  A.S_pad = S_pad; A.scale_log2e = scale * 1.4426950408889634f; A.nsplit = nsplit; A.nslot = nslot;
  A.n_kv = n_kv; A.n_q = n_q; A.G = n_q / n_kv; A.NB = NB;
  A.kt = (const u16*)kt; A.vt = (const u16*)vt; A.tl = TL; A.tcap = TCAP;
  A.epochs = epoch; A.out = (u16*)out;
  GAAC_REQUIRE(!epoch || out, "gaac_attn: the fused merge needs an output buffer");
  A.pool = nullptr; A.raw = nullptr; A.mt = nullptr; A.bt = nullptr; A.bt_stride = 0; A.TS = 0;
  A.freeq = nullptr; A.n_free = 0; A.stack = nullptr; A.top = nullptr;
#ifdef GAAC_PHASE_TIMING
  A.dbg = g_dbg;
#endif
  // few blocks: one 8-wave block per CU (half as many partials); otherwise two 4-wave blocks per CU
  const bool wide = (long)B * n_kv * nslot <= 256;
  const dim3 grid(B * n_kv * nslot), block(wide ? 512 : 256);
#ifdef GAAC_WAVES12
  if (wide && S_all >= 0) hipLaunchKernelGGL((k_attn_split<false, 12, true>), grid, dim3(768), 0, (hipStream_t)stream, A);
#else
  if (wide && S_all >= 0) hipLaunchKernelGGL((k_attn_split<false, 8, true>), grid, block, 0, (hipStream_t)stream, A);
#endif
  else if (wide) hipLaunchKernelGGL((k_attn_split<false, 8, false>), grid, block, 0, (hipStream_t)stream, A);
  else if (S_all >= 0) hipLaunchKernelGGL((k_attn_split<false, 4, true>), grid, block, 0, (hipStream_t)stream, A);
  else hipLaunchKernelGGL((k_attn_split<false, 4, false>), grid, block, 0, (hipStream_t)stream, A);
  return launch_status("gaac_attn(split)");
}

extern "C" int gaac_attn_split(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, float* pm, float* pl, float* pa, void* stream) {
  return attn_split_impl(smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v, q, slot, B, n_q, n_kv, SL, S_pad,
                         scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, nullptr, nullptr, -1, stream);
}

extern "C" int gaac_attn_combine(const float* pm, const float* pl, const float* pa, void* out, int n_rows, int nslot, void* stream) {
  GAAC_REQUIRE(pm && pl && pa && out && n_rows > 0 && nslot >= 1 && nslot <= MAX_SLOTS, "gaac_attn_combine: bad arguments");
  hipLaunchKernelGGL(k_attn_combine, dim3(n_rows), dim3(512), 0, (hipStream_t)stream, pm, pl, pa, (u16*)out, nslot);
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
                           scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, nullptr, nullptr, -1, stream);
  if (rc) return rc;
  return gaac_attn_combine(pm, pl, pa, out, B * n_q, nsplit, stream);
}

extern "C" int gaac_attn_fused(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, int S_all,
    unsigned long long* pm, unsigned long long* pl, unsigned long long* pa, unsigned int* epoch, void* out, void* stream) {
  GAAC_REQUIRE(out && epoch, "gaac_attn_fused: null output or epoch buffer");
  return attn_split_impl(smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v, q, slot, B, n_q, n_kv, SL, S_pad,
                         scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, epoch, out, S_all, stream);
}

// ---- the one entry point that allocates nothing ------------------------------------------------------------------------------------
// gaac_attn_fused with its workspace (partial records + epoch words) in a file-scope device array instead of caller memory, for callers
// that cannot allocate: code under HIP graph capture, tight serving loops.  Every GPU the library runs on holds its own copy of the
// array (4 MiB) from module load to process end; its address on a device comes from hipGetSymbolAddress, once per device
// (gaac_static_init, or the first call on that device outside stream capture).
constexpr size_t STATIC_SCRATCH_BYTES = 4u << 20;
constexpr long STATIC_MAX_RECORD_ROWS = 4000;                                               // B*n_q*nsplit (and so the grid's blocks) at most
constexpr size_t STATIC_EPOCH_BYTES = ((EPOCH_WORDS + STATIC_MAX_RECORD_ROWS) * sizeof(u32) + 255) / 256 * 256;      // epoch words + arrival marks
static_assert(STATIC_EPOCH_BYTES + STATIC_MAX_RECORD_ROWS * (D + 2) * sizeof(u64) <= STATIC_SCRATCH_BYTES, "the built-in workspace holds 4000 partial rows");
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];              // zero at module load: epoch 0, no records
constexpr int STATIC_MAX_DEVICES = 64;
static std::atomic<void*> g_scratch_ptr[STATIC_MAX_DEVICES];      // the array's address on each device (the name `scratch` is not one in host code)
static std::mutex g_scratch_mutex;

// The device a call runs on: the stream's own device when it has one, else the calling thread's current device.
static int static_device_of(hipStream_t stream, int* dev) {
  hipDevice_t d = -1;
  hipError_t e = stream ? hipStreamGetDevice(stream, &d) : hipGetDevice(&d);
  if (e != hipSuccess || d < 0 || d >= STATIC_MAX_DEVICES) return gaac::fail("gaac static workspace: no usable device (%s)", hipGetErrorString(e));
  *dev = (int)d;
  return 0;
}
// Resolves (once per device, under a lock) and returns the array's address on `dev`; dev must be the calling thread's current device.
static int static_scratch(int dev, bool may_resolve, unsigned char** base) {
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    if (!may_resolve)
      return gaac::fail("gaac_attn_fused_static: the built-in workspace of device %d has not been set up and the stream is capturing; "
                        "call gaac_static_init() once before the capture", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    p = g_scratch_ptr[dev].load(std::memory_order_relaxed);
    if (!p) {
      int cur = -1;
      hipError_t e = hipGetDevice(&cur);
      if (e != hipSuccess || cur != dev) return gaac::fail("gaac static workspace: device %d is not the calling thread's current device (%d)", dev, cur);
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || !p) return gaac::fail("gaac static workspace: hipGetSymbolAddress failed (%s)", hipGetErrorString(e));
      g_scratch_ptr[dev].store(p, std::memory_order_release);
    }
  }
  *base = static_cast<unsigned char*>(p);
  return 0;
}

extern "C" int gaac_static_init(void) {
  int dev = -1;
  if (int rc = static_device_of(nullptr, &dev)) return rc;
  unsigned char* base = nullptr;
  return static_scratch(dev, true, &base);
}

__global__ void __launch_bounds__(256) k_fill_zero(u32x4* __restrict__ p, long n16) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) p[i] = u32x4{0u, 0u, 0u, 0u};
}
// Re-arms the built-in workspace of the stream's device after a failed launch: epoch words and records back to zero, by a kernel (not
// a memset node, so the call may be captured).
extern "C" int gaac_static_reset(void* stream) {
  int dev = -1;
  if (int rc = static_device_of((hipStream_t)stream, &dev)) return rc;
  hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
  if (stream && hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess) cs = hipStreamCaptureStatusNone;
  unsigned char* base = nullptr;
  if (int rc = static_scratch(dev, cs == hipStreamCaptureStatusNone, &base)) return rc;
  const long n16 = (long)(STATIC_SCRATCH_BYTES / 16);
  hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)((n16 + 255) / 256)), dim3(256), 0, (hipStream_t)stream, reinterpret_cast<u32x4*>(base), n16);
  return launch_status("gaac_static_reset");
}
// Failure bits of the built-in workspace of the stream's device (see gaac_attn_fused), copied to *flags_out (device memory) on the stream.
extern "C" int gaac_static_flags(unsigned int* flags_out, void* stream) {
  GAAC_REQUIRE(flags_out, "gaac_static_flags: null output");
  int dev = -1;
  if (int rc = static_device_of((hipStream_t)stream, &dev)) return rc;
  unsigned char* base = nullptr;
  if (int rc = static_scratch(dev, true, &base)) return rc;
  hipError_t e = hipMemcpyAsync(flags_out, base + sizeof(unsigned int), sizeof(unsigned int), hipMemcpyDeviceToDevice, (hipStream_t)stream);
  if (e != hipSuccess) return gaac::fail("gaac_static_flags: %s", hipGetErrorString(e));
  return 0;
}

extern "C" int gaac_attn_fused_static(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, int S_all, void* out, void* stream) {
  GAAC_REQUIRE(out, "gaac_attn_fused_static: null output");
  GAAC_REQUIRE(B > 0 && n_q > 0 && nsplit >= 1, "gaac_attn_fused_static: bad sizes B=%d n_q=%d nsplit=%d", B, n_q, nsplit);
  const long rec_rows = (long)B * n_q * nsplit;
  GAAC_REQUIRE(rec_rows <= STATIC_MAX_RECORD_ROWS,
               "gaac_attn_fused_static: B*n_q*nsplit = %ld exceeds the %ld partial rows the built-in workspace (%zu bytes) holds; use gaac_attn_fused with caller memory",
               rec_rows, STATIC_MAX_RECORD_ROWS, STATIC_SCRATCH_BYTES);
  int dev = -1;
  if (int rc = static_device_of((hipStream_t)stream, &dev)) return rc;
  unsigned char* base = g_scratch_ptr[dev].load(std::memory_order_acquire) ? static_cast<unsigned char*>(g_scratch_ptr[dev].load(std::memory_order_acquire)) : nullptr;
  if (!base) {      // first call on this device: resolve the address now, unless the stream is capturing (no runtime query inside a capture)
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (stream && hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess) cs = hipStreamCaptureStatusNone;
    if (int rc = static_scratch(dev, cs == hipStreamCaptureStatusNone, &base)) return rc;
  }
  unsigned int* epoch = reinterpret_cast<unsigned int*>(base);
  unsigned long long* pm = reinterpret_cast<unsigned long long*>(base + STATIC_EPOCH_BYTES);
  unsigned long long* pl = pm + rec_rows;
  unsigned long long* pa = pl + rec_rows;
  return attn_split_impl(smk, ck, fk, tok, ovk, ohsk, b3k, b4k, smv, cv, fv, tov, ovv, ohsv, b3v, b4v, q, slot, B, n_q, n_kv, SL, S_pad,
                         scale, nsplit, NB, kt, vt, TL, TCAP, pm, pl, pa, epoch, out, S_all, stream);
}

extern "C" int gaac_paged_attn(
    const uint8_t* pool, int TS, const void* raw, const int* mt, const int* bt, int bt_stride, const int* seq_lens, int max_seq_len,
    const void* q, int B, int n_q, int n_kv, float scale, int nsplit,
    const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int NB,
    unsigned long long* pm, unsigned long long* pl, unsigned long long* pa, unsigned int* epoch, void* out,
    const int* freeq, int n_free, int* stack, int* top, void* stream) {
  GAAC_REQUIRE(n_kv > 0 && n_q > 0 && n_q % n_kv == 0 && n_q / n_kv <= GMAX, "GQA group size must be 1..%d (n_q=%d, n_kv=%d)", GMAX, n_q, n_kv);
  GAAC_REQUIRE(!freeq || (n_free > 0 && stack && top), "gaac_paged_attn: a free queue needs its length, the stack and its top");
  GAAC_REQUIRE(pool && raw && mt && bt && seq_lens && q && b3k && b4k && b3v && b4v && pm && pl && pa && epoch && out, "gaac_paged_attn: null pointer");
  GAAC_REQUIRE(B > 0 && NB > 0 && TS >= SLOT_OV + 16 && TS % 16 == 0 && bt_stride > 0, "gaac_paged_attn: bad sizes B=%d NB=%d TS=%d (a slot is %d bytes plus at least 16 for escapes)", B, NB, TS, SLOT_OV);
  GAAC_REQUIRE(nsplit >= 1 && nsplit <= MAX_SLOTS, "gaac_paged_attn: nsplit must be in 1..%d", MAX_SLOTS);
  const long max_tiles = ((long)max_seq_len + T - 1) / T;
  GAAC_REQUIRE(max_seq_len >= 0 && max_tiles <= (long)bt_stride, "gaac_paged_attn: max_seq_len %d needs %ld blocks per row, the block table has %d", max_seq_len, max_tiles, bt_stride);
  AttnArgs A;
  A.k = StoreView{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, b3k, b4k};
  A.v = StoreView{nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, b3v, b4v};
  A.q = (const u16*)q; A.pm = (float*)pm; A.pl = (float*)pl; A.pa = (float*)pa; A.slot = nullptr; A.sl = seq_lens; A.S_all = -1;
  A.S_pad = 0; A.scale_log2e = scale * 1.4426950408889634f; A.nsplit = nsplit; A.nslot = nsplit;
  A.n_kv = n_kv; A.n_q = n_q; A.G = n_q / n_kv; A.NB = NB;
  A.kt = nullptr; A.vt = nullptr; A.tl = nullptr; A.tcap = 0;
  A.epochs = epoch; A.out = (u16*)out;
  A.pool = pool; A.raw = (const u16*)raw; A.mt = mt; A.bt = bt; A.bt_stride = bt_stride; A.TS = TS;
  A.freeq = freeq; A.n_free = freeq ? n_free : 0; A.stack = stack; A.top = top;
#ifdef GAAC_PHASE_TIMING
  A.dbg = g_dbg;
#endif
  if ((long)B * n_kv * nsplit <= 256) hipLaunchKernelGGL((k_attn_split<true, 8, false>), dim3(B * n_kv * nsplit), dim3(512), 0, (hipStream_t)stream, A);
  else hipLaunchKernelGGL((k_attn_split<true, 4, false>), dim3(B * n_kv * nsplit), dim3(256), 0, (hipStream_t)stream, A);
  return launch_status("gaac_paged_attn");
}

extern "C" int gaac_bf16_attn(const void* k, const void* v, int S, const int* seq_lens, long head_stride_tokens, const void* q, int B, int n_q,
                              int n_kv, float scale, int nsplit, unsigned long long* pm, unsigned long long* pl, unsigned long long* pa,
                              unsigned int* epoch, void* out, void* stream) {
  GAAC_REQUIRE(n_kv > 0 && n_q > 0 && n_q % n_kv == 0 && n_q / n_kv <= GMAX, "GQA group size must be 1..%d (n_q=%d, n_kv=%d)", GMAX, n_q, n_kv);
  GAAC_REQUIRE(k && v && q && pm && pl && pa && epoch && out, "gaac_bf16_attn: null pointer");
  GAAC_REQUIRE(B > 0 && S > 0 && head_stride_tokens >= S && nsplit >= 1 && nsplit <= MAX_SLOTS, "gaac_bf16_attn: bad sizes");
  AttnArgs A = {};
  A.q = (const u16*)q; A.pm = (float*)pm; A.pl = (float*)pl; A.pa = (float*)pa; A.S_all = -1;
  A.S_pad = (int)head_stride_tokens; A.scale_log2e = scale * 1.4426950408889634f; A.nsplit = nsplit; A.nslot = nsplit;
  A.n_kv = n_kv; A.n_q = n_q; A.G = n_q / n_kv; A.NB = 1;
  A.kt = (const u16*)k; A.vt = (const u16*)v; A.tcap = S; A.sl = seq_lens;
  A.epochs = epoch; A.out = (u16*)out;
  if ((long)B * n_kv * nsplit <= 256) hipLaunchKernelGGL(k_bf16_attn_split<8>, dim3(B * n_kv * nsplit), dim3(512), 0, (hipStream_t)stream, A);
  else hipLaunchKernelGGL(k_bf16_attn_split<4>, dim3(B * n_kv * nsplit), dim3(256), 0, (hipStream_t)stream, A);
  return launch_status("gaac_bf16_attn");
}
