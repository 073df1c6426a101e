// Paged slot pool: store path, raw-tile free list and block decode.  Counterpart of /root/reference/gaac/vllm/store.py:22-174
// (_store_tiles, _free_tiles, _decode_tiles, _release_blocks) with the slot geometry of store.py:17-19 and paged_kernel.py:3-6:
//
//   block (16 tokens, all kv heads, K and V) = 2*n_kv tile slots of TS bytes, slot t = 2*kvh + kind, physical tile p = blk*2*n_kv + t
//   slot = [0,2048) sign/mantissa | [2048,2816) codes | [2816,2880) 16 tag words | [2880,TS) escape bytes (OVF_SLOT = TS - 2880)
//   mode table MT[p] = p  -> compressed in its slot;  ~r -> raw BF16 tile r of the side pool RAW[r][16][128] (a block that is still
//   filling, or a finished tile whose escape bytes do not fit the slot).
// Sign/mantissa and code bytes inside a slot are in the native tile order of gaac_core.h; raw tiles are in natural channel order.
// One wave per (store entry, tile slot).  Pops of the free stack happen only in k_paged_store and pushes only in k_paged_free /
// k_paged_release, which are separate launches, so a pop never races a push.
#include "gaac_tile.h"
#include "gaac_capi.h"

namespace gaac {

constexpr int SLOT_CD = TILE_SM, SLOT_FL = TILE_SM + TILE_CD, SLOT_OV = SLOT_FL + 4 * T;      // 2048, 2816, 2880

struct PagedStoreArgs {
  const u16* key; const u16* value; long k_stride, v_stride;      // rows [num_tokens][n_kv][128] bf16, row stride in elements
  const int* ent; int n_ent;                                       // [E][4] = (block, first token row, block offset, rows); block < 0: inactive
  uint8_t* pool; int TS; u16* raw; int* mt; int* stack; int* top; int* err; int* freeq;
  const uint8_t* b3k; const uint8_t* b4k; const uint8_t* b3v; const uint8_t* b4v;
  int n_kv, ovf_slot;
};

// pops one raw tile; -1 (and the error counter goes up) when the side pool is empty.  Uniform result for the wave.
__device__ __forceinline__ int pop_raw_tile(const PagedStoreArgs& A, int lane) {
  int r = -1;
  if (lane == 0) {
    const int idx = atomicSub(A.top, 1) - 1;
    if (idx >= 0) r = A.stack[idx];
    else { atomicAdd(A.top, 1); atomicAdd(A.err, 1); }
  }
  return __builtin_amdgcn_readfirstlane(r);
}

template <int KIND>
__device__ __forceinline__ void store_tile(const PagedStoreArgs& A, EncodeLds& L, int e, int t, int kvh, int lane) {
  const int blk = A.ent[4 * e], tok0 = A.ent[4 * e + 1], off0 = A.ent[4 * e + 2], n = A.ent[4 * e + 3];
  const int qi = e * 2 * A.n_kv + t;
  if (blk < 0 || n <= 0 || off0 < 0 || off0 + n > T) { if (lane == 0) A.freeq[qi] = -1; return; }
  const long p = (long)blk * (2 * A.n_kv) + t;
  const int old = A.mt[p];
  const bool have = old < 0;
  const int r_old = have ? ~old : -1;
  const bool full = off0 + n == T;
  const u16* src = (KIND == KIND_K ? A.key : A.value) + (long)kvh * D;
  const long stride = KIND == KIND_K ? A.k_stride : A.v_stride;
  bool fits = false;
  if (full) {
    // gather the tile: rows below off0 from the raw tile of the block, the rest from this step's rows
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int idx = k * 64 + lane, row = idx >> 4, c16 = idx & 15;
      u32x4 v = {0u, 0u, 0u, 0u};
      if (row >= off0) v = *reinterpret_cast<const u32x4*>(src + (long)(tok0 + row - off0) * stride + c16 * 8);
      else if (have) v = *reinterpret_cast<const u32x4*>(A.raw + ((long)r_old * T + row) * D + c16 * 8);
      *reinterpret_cast<u32x4*>(&L.x[row * XROW + c16 * 8]) = v;
    }
    stage_bases(L, (KIND == KIND_K ? A.b3k : A.b3v) + (long)kvh * D, (KIND == KIND_K ? A.b4k : A.b4v) + (long)kvh * D, lane);
    wave_lds_sync();
    BaseRegs Bs;
    load_base_regs<KIND>(L, lane & 15, lane >> 4, Bs);
    uint8_t* slot = A.pool + p * A.TS;
    const int total = encode_staged_tile<KIND>(L, Bs, T, lane, slot, slot + SLOT_CD, reinterpret_cast<int*>(slot + SLOT_FL), nullptr);
    fits = total <= A.ovf_slot;
    if (fits) encode_staged_tile<KIND>(L, Bs, T, lane, slot, slot + SLOT_CD, reinterpret_cast<int*>(slot + SLOT_FL), slot + SLOT_OV);
  }
  int r = r_old;
  if (!fits) {      // the rows stay raw: a filling block, or a finished tile whose escapes exceed the slot
    if (!have) r = pop_raw_tile(A, lane);
    if (r >= 0) {
      for (int idx = lane; idx < n * 16; idx += 64) {
        const int row = idx >> 4, c16 = idx & 15;
        *reinterpret_cast<u32x4*>(A.raw + ((long)r * T + off0 + row) * D + c16 * 8) =
            *reinterpret_cast<const u32x4*>(src + (long)(tok0 + row) * stride + c16 * 8);
      }
    }
  }
  if (!fits && r < 0 && lane < T) {
    // side pool exhausted: the slot will read as a compressed tile with stale content (the error counter says so).  Its tag words must
    // not send a reader past the slot: the size pass above, or an earlier tenant of the block, may have left tags whose escape bytes
    // (up to 1280) exceed the slot's capacity.  All-zero tags mean no escape bytes.
    reinterpret_cast<int*>(A.pool + p * A.TS + SLOT_FL)[lane] = 0;
  }
  if (lane == 0) {
    A.mt[p] = fits || r < 0 ? (int)p : ~r;         // pool exhausted: the slot reads as a (stale) compressed tile, the error counter says so
    A.freeq[qi] = fits && have ? r_old : -1;        // a raw tile that is no longer needed goes back after this launch
  }
}

// grid (E, 2*n_kv), one wave each
__global__ void __launch_bounds__(64) k_paged_store(const PagedStoreArgs A) {
  __shared__ EncodeLds L;
  const int e = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
  if (t & 1) store_tile<KIND_V>(A, L, e, t, t >> 1, lane);
  else store_tile<KIND_K>(A, L, e, t, t >> 1, lane);
}

__global__ void __launch_bounds__(256) k_paged_free(const int* __restrict__ freeq, int n_items, int* __restrict__ stack, int* __restrict__ top) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n_items) return;
  const int r = freeq[i];
  if (r >= 0) stack[atomicAdd(top, 1)] = r;
}

// blocks whose content is dead: their raw tiles go back to the free stack and the mode table is reset (store.py:164-174)
__global__ void __launch_bounds__(64) k_paged_release(const int* __restrict__ blocks, int* __restrict__ mt, int* __restrict__ stack,
                                                      int* __restrict__ top, int nt) {
  const int blk = blocks[blockIdx.x];
  if (blk < 0) return;
  for (int t = threadIdx.x; t < nt; t += 64) {
    const long p = (long)blk * nt + t;
    const int m = mt[p];
    if (m < 0) { stack[atomicAdd(top, 1)] = ~m; mt[p] = (int)p; }
  }
}

struct PagedDecodeArgs {
  const uint8_t* pool; int TS; const u16* raw; const int* mt; const int* pairs;      // pairs [P][3] = (block, first output row, valid rows)
  u16* sk; u16* sv; long row_stride;
  const uint8_t* b3k; const uint8_t* b4k; const uint8_t* b3v; const uint8_t* b4v; int n_kv;
};
// grid (P, 2*n_kv), one wave each: expands one (block, tile slot) into BF16 rows of a flat K / V [rows, n_kv, 128] (store.py:117-161)
__global__ void __launch_bounds__(64) k_paged_decode(const PagedDecodeArgs A) {
  const int e = blockIdx.x, t = blockIdx.y, lane = threadIdx.x, kind = t & 1, kvh = t >> 1;
  const int blk = A.pairs[3 * e], row0 = A.pairs[3 * e + 1], nvalid = min(A.pairs[3 * e + 2], T);
  if (blk < 0 || nvalid <= 0) return;
  const long p = (long)blk * (2 * A.n_kv) + t;
  const int m = A.mt[p];
  u16* out = (kind ? A.sv : A.sk) + (long)row0 * A.row_stride + (long)kvh * D;
  if (m < 0) {
    const u16* src = A.raw + (long)(~m) * T * D;
    for (int idx = lane; idx < nvalid * 16; idx += 64) {
      const int row = idx >> 4, c16 = idx & 15;
      *reinterpret_cast<u32x4*>(out + (long)row * A.row_stride + c16 * 8) = *reinterpret_cast<const u32x4*>(src + row * D + c16 * 8);
    }
    return;
  }
  const uint8_t* slot = A.pool + (long)m * A.TS;
  __shared__ __align__(16) u16 stage[T * STAGE_ROW];
  const bool aligned = (A.row_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
  if (kind) {
    if (aligned) decode_tile_staged<KIND_V>(slot, slot + SLOT_CD, reinterpret_cast<const int*>(slot + SLOT_FL), slot + SLOT_OV,
                                            A.b3v + (long)kvh * D, A.b4v + (long)kvh * D, lane, nvalid, stage, out, A.row_stride);
    else decode_tile_rows<KIND_V>(slot, slot + SLOT_CD, reinterpret_cast<const int*>(slot + SLOT_FL), slot + SLOT_OV,
                                  A.b3v + (long)kvh * D, A.b4v + (long)kvh * D, lane, nvalid, out, A.row_stride);
  } else {
    if (aligned) decode_tile_staged<KIND_K>(slot, slot + SLOT_CD, reinterpret_cast<const int*>(slot + SLOT_FL), slot + SLOT_OV,
                                            A.b3k + (long)kvh * D, A.b4k + (long)kvh * D, lane, nvalid, stage, out, A.row_stride);
    else decode_tile_rows<KIND_K>(slot, slot + SLOT_CD, reinterpret_cast<const int*>(slot + SLOT_FL), slot + SLOT_OV,
                                  A.b3k + (long)kvh * D, A.b4k + (long)kvh * D, lane, nvalid, out, A.row_stride);
  }
}

}  // namespace gaac

using namespace gaac;

extern "C" {

int gaac_paged_store(const void* key, const void* value, long k_stride, long v_stride, const int* ent, int n_ent,
                     uint8_t* pool, int TS, void* raw, int* mt, int* stack, int* top, int* err, int* freeq,
                     const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int n_kv, void* stream) {
  GAAC_REQUIRE(key && value && ent && pool && raw && mt && stack && top && err && freeq && b3k && b4k && b3v && b4v, "gaac_paged_store: null pointer");
  GAAC_REQUIRE(n_ent > 0 && n_kv > 0 && TS >= SLOT_OV + 16 && TS % 16 == 0 && k_stride >= (long)n_kv * D && v_stride >= (long)n_kv * D,
               "gaac_paged_store: bad sizes n_ent=%d n_kv=%d TS=%d", n_ent, n_kv, TS);
  PagedStoreArgs A{(const u16*)key, (const u16*)value, k_stride, v_stride, ent, n_ent, pool, TS, (u16*)raw, mt, stack, top, err, freeq,
                   b3k, b4k, b3v, b4v, n_kv, TS - SLOT_OV};
  hipLaunchKernelGGL(k_paged_store, dim3(n_ent, 2 * n_kv), dim3(64), 0, (hipStream_t)stream, A);
  return launch_status("gaac_paged_store");
}

int gaac_paged_free(const int* freeq, int n_items, int* stack, int* top, void* stream) {
  GAAC_REQUIRE(freeq && stack && top && n_items > 0, "gaac_paged_free: bad arguments");
  hipLaunchKernelGGL(k_paged_free, dim3((n_items + 255) / 256), dim3(256), 0, (hipStream_t)stream, freeq, n_items, stack, top);
  return launch_status("gaac_paged_free");
}

int gaac_paged_release(const int* blocks, int n_blocks, int* mt, int* stack, int* top, int n_kv, void* stream) {
  GAAC_REQUIRE(blocks && mt && stack && top && n_blocks > 0 && n_kv > 0, "gaac_paged_release: bad arguments");
  hipLaunchKernelGGL(k_paged_release, dim3(n_blocks), dim3(64), 0, (hipStream_t)stream, blocks, mt, stack, top, 2 * n_kv);
  return launch_status("gaac_paged_release");
}

int gaac_paged_decode(const uint8_t* pool, int TS, const void* raw, const int* mt, const int* pairs, int n_pairs, void* sk, void* sv,
                      long row_stride, const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int n_kv, void* stream) {
  GAAC_REQUIRE(pool && raw && mt && pairs && sk && sv && b3k && b4k && b3v && b4v, "gaac_paged_decode: null pointer");
  GAAC_REQUIRE(n_pairs > 0 && n_kv > 0 && TS >= SLOT_OV + 16 && TS % 16 == 0 && row_stride >= (long)n_kv * D, "gaac_paged_decode: bad sizes");
  PagedDecodeArgs A{pool, TS, (const u16*)raw, mt, pairs, (u16*)sk, (u16*)sv, row_stride, b3k, b4k, b3v, b4v, n_kv};
  hipLaunchKernelGGL(k_paged_decode, dim3(n_pairs, 2 * n_kv), dim3(64), 0, (hipStream_t)stream, A);
  return launch_status("gaac_paged_decode");
}

}  // extern "C"
