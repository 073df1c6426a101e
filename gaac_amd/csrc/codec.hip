// Calibration, page encoder and page decoder kernels + their extern "C" entry points.
//   exponent_hist / bases_from_hist   /root/reference/gaac/codec.py:70-84
//   encode_tiles / compact            /root/reference/gaac/encoder.py:16-76, 94-109
//   row_offsets                       /root/reference/gaac/codec.py:221-225
//   decode_tiles                      /root/reference/gaac/codec.py:186-218
#include "gaac_tile.h"
#include "gaac_capi.h"
#include "../../include/gaac_hip.h"

namespace gaac {

char* last_error_buffer() { static thread_local char buf[512] = {0}; return buf; }

// ---------------------------------------------------------------------------------------------------- calibration
// Exponent histogram per (kv head, channel).  A block owns 64 channels of the n_kv*128-wide token row and a chunk of tokens: eight
// lanes read the 128 bytes of a row with 16-byte loads, counts go to LDS (64 x 256 x 4 B) and from there, where non-zero, to the
// 64-bit global histogram.
constexpr int HIST_CH = 64;
__global__ void __launch_bounds__(256) k_exponent_hist(const u16* __restrict__ x, long n_tok, int n_kv, int chunk,
                                                       unsigned long long* __restrict__ hist) {
  __shared__ u32 h[HIST_CH * 256];
  const int tid = threadIdx.x, c0 = blockIdx.x * HIST_CH;      // first of this block's channels in the n_kv*128 row
  for (int i = tid; i < HIST_CH * 256; i += 256) h[i] = 0u;
  __syncthreads();
  const long t0 = (long)blockIdx.y * chunk, t1 = min(t0 + (long)chunk, n_tok);
  const int c8 = tid & 7, sub = tid >> 3;
  const long row = (long)n_kv * D;
  const u16* xp = x + c0 + 8 * c8;
  u32* hc = h + (8 * c8) * 256;
  for (long t = t0 + sub; t < t1; t += 4 * 32) {      // four rows in flight per thread
    u32x4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) v[k] = t + 32 * k < t1 ? *reinterpret_cast<const u32x4*>(xp + (t + 32 * k) * row) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (t + 32 * k >= t1) break;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        atomicAdd(&hc[(2 * j) * 256 + ((v[k][j] >> 7) & 0xFFu)], 1u);
        atomicAdd(&hc[(2 * j + 1) * 256 + ((v[k][j] >> 23) & 0xFFu)], 1u);
      }
    }
  }
  __syncthreads();
  for (int i = tid; i < HIST_CH * 256; i += 256)
    if (h[i]) atomicAdd(&hist[(long)(c0 + (i >> 8)) * 256 + (i & 255)], (unsigned long long)h[i]);
}

// One wave per histogram row: lane l evaluates the windows that start at 4l .. 4l+3 (the reference takes the first maximum of the
// window sums, codec.py:70-77: the lowest start wins ties).
__global__ void __launch_bounds__(256) k_bases_from_hist(const long long* __restrict__ hist, int rows,
                                                         uint8_t* __restrict__ base3, uint8_t* __restrict__ base4) {
  __shared__ long long hs[4][256 + 16];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = blockIdx.x * 4 + wave;
  if (r >= rows) return;
  long long* hr = hs[wave];
#pragma unroll
  for (int k = 0; k < 4; ++k) hr[lane + 64 * k] = hist[(long)r * 256 + lane + 64 * k];
  if (lane < 16) hr[256 + lane] = 0;
  wave_lds_sync();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int w = pass ? 16 : 8;
    long long best = -1; int arg = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int st = 4 * lane + j;
      long long sum = 0;
      for (int i = 0; i < w; ++i) sum += hr[st + i];
      if (st + w <= 256 && sum > best) { best = sum; arg = st; }
    }
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {      // maximum, lowest start among equals
      const long long ob = __shfl_xor(best, o, 64); const int oa = __shfl_xor(arg, o, 64);
      if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
    }
    if (lane == 0) (pass ? base4 : base3)[r] = (uint8_t)arg;
  }
}

// ---------------------------------------------------------------------------------------------------- page encoder
// A block of four waves takes 16 consecutive tiles of one head, wave w the tiles w, w+4, w+8, w+12 of them (one-wave blocks, one per
// tile, would be limited by the rate at which workgroups can be launched).  The rows of a wave's next tile are fetched into
// registers while it encodes the current one.
constexpr int CODEC_WAVES = 4, CODEC_TPW = 4, CODEC_TPB = CODEC_WAVES * CODEC_TPW;
template <int KIND>
__global__ void __launch_bounds__(64 * CODEC_WAVES) k_encode_tiles(const u16* __restrict__ x, int S, long x_head_stride, long x_row_stride, int S_pad,
                                                                   const uint8_t* __restrict__ base3, const uint8_t* __restrict__ base4,
                                                                   int n_kv, const int* __restrict__ bidx, uint8_t* __restrict__ sm,
                                                                   uint8_t* __restrict__ cd, int* __restrict__ flags,
                                                                   uint8_t* __restrict__ esc_slots, int* __restrict__ tile_bytes, int ntiles) {
  __shared__ EncodeLds Ls[CODEC_WAVES];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, h = blockIdx.y;
  EncodeLds& L = Ls[wave];
  const int brow = bidx ? bidx[h] : h % n_kv;
  int tile = blockIdx.x * CODEC_TPB + wave;
  if (tile >= ntiles) return;
  const u16* xh = x + (long)h * x_head_stride;
  RowRegs R, Rn;
  load_rows(R, xh + (long)tile * T * x_row_stride, x_row_stride, min(T, S - tile * T), lane);
  stage_bases(L, base3 + (long)brow * D, base4 + (long)brow * D, lane);
  wave_lds_sync();
  BaseRegs Bs;                // the base words of the lane's units: the same for every tile of the head
  load_base_regs<KIND>(L, lane & 15, lane >> 4, Bs);
  for (int i = 0; i < CODEC_TPW && tile < ntiles; ++i, tile += CODEC_WAVES) {
    const int nvalid = min(T, S - tile * T), next = tile + CODEC_WAVES;
    store_rows(L, R, lane);
    if (i + 1 < CODEC_TPW && next < ntiles) load_rows(Rn, xh + (long)next * T * x_row_stride, x_row_stride, min(T, S - next * T), lane);
    wave_lds_sync();
    const long row0 = (long)h * S_pad + (long)tile * T;
    const int total = encode_staged_tile<KIND>(L, Bs, nvalid, lane, sm + row0 * D, cd + row0 * CB, flags + row0,
                                               esc_slots + ((long)h * ntiles + tile) * TILE_MAX_ESC);
    if (lane == 0) tile_bytes[(long)h * ntiles + tile] = total;
    wave_lds_sync();          // the staged rows and tag words are free again
    R = Rn;
  }
}

// Packs the per-tile escape slots into the head's stream and writes the tile offsets (exclusive sum of the tile sizes of the head).
// A block takes 64 consecutive tiles: it sums the sizes of all earlier tiles of the head itself (a few thousand integers at most),
// scans its own 64 and copies, one wave per tile: most tiles hold a few dozen escape bytes.
constexpr int COMPACT_TPB = 64;
__global__ void __launch_bounds__(256) k_compact(const uint8_t* __restrict__ esc_slots, const int* __restrict__ tile_bytes,
                                                 int* __restrict__ tile_off, const int* __restrict__ head_start,
                                                 uint8_t* __restrict__ ovf, int ntiles) {
  __shared__ int part[4];
  __shared__ int offs[COMPACT_TPB];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, h = blockIdx.y, t0 = blockIdx.x * COMPACT_TPB;
  const int* tb = tile_bytes + (long)h * ntiles;
  int before = 0;
  for (int i = tid; i < t0; i += 256) before += tb[i];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) before += __shfl_xor(before, o, 64);
  if (lane == 0) part[wave] = before;
  __syncthreads();
  if (wave == 0) {
    const int n = t0 + lane < ntiles ? tb[t0 + lane] : 0;
    int incl = n;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { const int v = __shfl_up(incl, o, 64); if (lane >= o) incl += v; }
    const int off = part[0] + part[1] + part[2] + part[3] + incl - n;
    offs[lane] = off;
    if (t0 + lane < ntiles) tile_off[(long)h * ntiles + t0 + lane] = off;
  }
  __syncthreads();
  const int hs = head_start[h];
  for (int k = wave; k < COMPACT_TPB && t0 + k < ntiles; k += 4) {
    const long i = (long)h * ntiles + t0 + k;
    const int n = tb[t0 + k];
    const uint8_t* src = esc_slots + i * TILE_MAX_ESC;
    uint8_t* dst = ovf + hs + offs[k];
    for (int j = lane; j < n; j += 64) dst[j] = src[j];
  }
}

// Two passes over the tag words of a head: escape bytes per chunk of 2048 rows, then per chunk the bytes of all earlier chunks (a
// short sum) plus a scan inside the chunk: 8 words per thread serially, thread totals by a block scan.
constexpr int RO_CHUNK = 2048;
__global__ void __launch_bounds__(256) k_row_chunk_sums(const int* __restrict__ flags, int S, int S_pad, int* __restrict__ chunk_sums) {
  __shared__ int sh[4];
  const int h = blockIdx.y, c = blockIdx.x, tid = threadIdx.x;
  const int* f = flags + (long)h * S_pad;
  const int s0 = c * RO_CHUNK + tid * 8;
  int mine = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) mine += s0 + k < S ? esc_bytes((u32)f[s0 + k]) : 0;
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mine += __shfl_xor(mine, o, 64);
  if ((tid & 63) == 0) sh[tid >> 6] = mine;
  __syncthreads();
  if (tid == 0) chunk_sums[(long)h * gridDim.x + c] = sh[0] + sh[1] + sh[2] + sh[3];
}
__global__ void __launch_bounds__(256) k_row_offsets(const int* __restrict__ flags, int S, int S_pad, const int* __restrict__ chunk_sums,
                                                     int* __restrict__ out) {
  __shared__ int sh[256];
  const int h = blockIdx.y, c = blockIdx.x, tid = threadIdx.x;
  const int* f = flags + (long)h * S_pad;
  int before = 0;
  for (int i = tid; i < c; i += 256) before += chunk_sums[(long)h * gridDim.x + i];
  const int s0 = c * RO_CHUNK + tid * 8;
  int rb[8], mine = 0;
#pragma unroll
  for (int k = 0; k < 8; ++k) { rb[k] = s0 + k < S ? esc_bytes((u32)f[s0 + k]) : 0; mine += rb[k]; }
  // block-wide: sum of `before`, inclusive scan of `mine`
  sh[tid] = before;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) { if (tid < o) sh[tid] += sh[tid + o]; __syncthreads(); }
  const int base = sh[0];
  __syncthreads();
  sh[tid] = mine;
  __syncthreads();
  for (int o = 1; o < 256; o <<= 1) {
    const int v = tid >= o ? sh[tid - o] : 0;
    __syncthreads();
    sh[tid] += v;
    __syncthreads();
  }
  int off = base + sh[tid] - mine;
#pragma unroll
  for (int k = 0; k < 8; ++k) { if (s0 + k < S) out[(long)h * S + s0 + k] = off; off += rb[k]; }
}

// ---------------------------------------------------------------------------------------------------- page decoder
// One wave per tile: short-lived waves at full occupancy overlap the dependent loads of a tile (tag words -> escape bytes) with the
// arithmetic and the stores of others (four tiles in a row per wave were a third slower).
template <int KIND>
__global__ void __launch_bounds__(64) k_decode_tiles(const uint8_t* __restrict__ sm, const uint8_t* __restrict__ cd, const int* __restrict__ flags,
                                                     const int* __restrict__ tile_off, const uint8_t* __restrict__ ovf,
                                                     const int* __restrict__ head_start, const uint8_t* __restrict__ base3,
                                                     const uint8_t* __restrict__ base4, int n_kv, const int* __restrict__ bidx,
                                                     int S, int S_pad, u16* __restrict__ out, long out_head_stride, long out_row_stride) {
  const int tile = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int brow = bidx ? bidx[h] : h % n_kv;
  const long row0 = (long)h * S_pad + (long)tile * T;
  // rows beyond S carry tag 0 (the encoder writes every word of a tile) and are not written
  __shared__ __align__(16) u16 stage[T * STAGE_ROW];
  u16* dst = out + (long)h * out_head_stride + (long)tile * T * out_row_stride;
  const uint8_t* esc = ovf + head_start[h] + tile_off[(long)h * (S_pad / T) + tile];
  if ((out_row_stride & 7) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15) == 0)
    decode_tile_staged<KIND>(sm + row0 * D, cd + row0 * CB, flags + row0, esc, base3 + (long)brow * D, base4 + (long)brow * D, lane,
                             min(T, S - tile * T), stage, dst, out_row_stride);
  else      // rows that are not 16-byte aligned: element stores
    decode_tile_rows<KIND>(sm + row0 * D, cd + row0 * CB, flags + row0, esc, base3 + (long)brow * D, base4 + (long)brow * D, lane,
                           min(T, S - tile * T), dst, out_row_stride);
}

}  // namespace gaac

using namespace gaac;

extern "C" {

const char* gaac_last_error(void) { return last_error_buffer(); }

int gaac_exponent_hist(const void* x, long n_tokens, int n_kv, long long* hist, void* stream) {
  GAAC_REQUIRE(x && hist && n_kv > 0 && n_tokens >= 0, "gaac_exponent_hist: bad arguments");
  if (n_tokens == 0) return 0;
  int nchunk = (int)min((n_tokens + 1023) / 1024, 512L);
  int chunk = (int)((n_tokens + nchunk - 1) / nchunk);
  hipLaunchKernelGGL(k_exponent_hist, dim3(n_kv * D / HIST_CH, nchunk), dim3(256), 0, (hipStream_t)stream,
                     (const u16*)x, n_tokens, n_kv, chunk, (unsigned long long*)hist);
  return launch_status("gaac_exponent_hist");
}

int gaac_bases_from_hist(const long long* hist, int rows, uint8_t* base3, uint8_t* base4, void* stream) {
  GAAC_REQUIRE(hist && base3 && base4 && rows > 0, "gaac_bases_from_hist: bad arguments");
  hipLaunchKernelGGL(k_bases_from_hist, dim3((rows + 3) / 4), dim3(256), 0, (hipStream_t)stream, hist, rows, base3, base4);
  return launch_status("gaac_bases_from_hist");
}

int gaac_encode_tiles(int kind, const void* x, long x_head_stride, long x_row_stride, int H, int S, int S_pad, const uint8_t* base3,
                      const uint8_t* base4, int n_kv, const int* bidx, uint8_t* sm, uint8_t* codes, int* flags, uint8_t* esc_slots,
                      int* tile_bytes, void* stream) {
  GAAC_REQUIRE(kind == 0 || kind == 1, "gaac_encode_tiles: kind must be 0 (k) or 1 (v)");
  GAAC_REQUIRE(x && base3 && base4 && sm && codes && flags && esc_slots && tile_bytes, "gaac_encode_tiles: null pointer");
  GAAC_REQUIRE(H > 0 && S > 0 && S_pad >= (S + T - 1) / T * T && S_pad % T == 0 && n_kv > 0,
               "gaac_encode_tiles: bad sizes H=%d S=%d S_pad=%d n_kv=%d", H, S, S_pad, n_kv);
  GAAC_REQUIRE(x_row_stride >= D && x_row_stride % 8 == 0 && x_head_stride % 8 == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0,
               "gaac_encode_tiles: rows must be 16-byte aligned (strides in elements: head %ld, row %ld)", x_head_stride, x_row_stride);
  const int ntiles = (S + T - 1) / T;
  dim3 grid((ntiles + CODEC_TPB - 1) / CODEC_TPB, H);
  if (kind == 0) hipLaunchKernelGGL(k_encode_tiles<KIND_K>, grid, dim3(64 * CODEC_WAVES), 0, (hipStream_t)stream, (const u16*)x, S, x_head_stride, x_row_stride, S_pad, base3, base4, n_kv, bidx, sm, codes, flags, esc_slots, tile_bytes, ntiles);
  else hipLaunchKernelGGL(k_encode_tiles<KIND_V>, grid, dim3(64 * CODEC_WAVES), 0, (hipStream_t)stream, (const u16*)x, S, x_head_stride, x_row_stride, S_pad, base3, base4, n_kv, bidx, sm, codes, flags, esc_slots, tile_bytes, ntiles);
  return launch_status("gaac_encode_tiles");
}

int gaac_compact(const uint8_t* esc_slots, const int* tile_bytes, int* tile_off, const int* head_start, uint8_t* ovf,
                 int H, int ntiles, void* stream) {
  GAAC_REQUIRE(esc_slots && tile_bytes && tile_off && head_start && ovf && H > 0 && ntiles > 0, "gaac_compact: bad arguments");
  hipLaunchKernelGGL(k_compact, dim3((ntiles + COMPACT_TPB - 1) / COMPACT_TPB, H), dim3(256), 0, (hipStream_t)stream, esc_slots, tile_bytes, tile_off, head_start, ovf, ntiles);
  return launch_status("gaac_compact");
}

int gaac_row_offsets(const int* flags, int H, int S, int S_pad, int* chunk_sums, int* out, void* stream) {
  GAAC_REQUIRE(flags && out && chunk_sums && H > 0 && S > 0 && S_pad >= S, "gaac_row_offsets: bad arguments");
  const dim3 grid((S + RO_CHUNK - 1) / RO_CHUNK, H);
  hipLaunchKernelGGL(k_row_chunk_sums, grid, dim3(256), 0, (hipStream_t)stream, flags, S, S_pad, chunk_sums);
  hipLaunchKernelGGL(k_row_offsets, grid, dim3(256), 0, (hipStream_t)stream, flags, S, S_pad, chunk_sums, out);
  return launch_status("gaac_row_offsets");
}

int gaac_decode_tiles(int kind, const uint8_t* sm, const uint8_t* codes, const int* flags, const int* tile_off, const uint8_t* ovf,
                      const int* head_start, const uint8_t* base3, const uint8_t* base4, int n_kv, const int* bidx, int H, int S,
                      int S_pad, void* out, long out_head_stride, long out_row_stride, void* stream) {
  GAAC_REQUIRE(kind == 0 || kind == 1, "gaac_decode_tiles: kind must be 0 (k) or 1 (v)");
  GAAC_REQUIRE(sm && codes && flags && tile_off && ovf && head_start && base3 && base4 && out, "gaac_decode_tiles: null pointer");
  GAAC_REQUIRE(H > 0 && S > 0 && S_pad >= (S + T - 1) / T * T && S_pad % T == 0 && n_kv > 0, "gaac_decode_tiles: bad sizes");
  dim3 grid((S + T - 1) / T, H);
  if (kind == 0) hipLaunchKernelGGL(k_decode_tiles<KIND_K>, grid, dim3(64), 0, (hipStream_t)stream, sm, codes, flags, tile_off, ovf, head_start, base3, base4, n_kv, bidx, S, S_pad, (u16*)out, out_head_stride, out_row_stride);
  else hipLaunchKernelGGL(k_decode_tiles<KIND_V>, grid, dim3(64), 0, (hipStream_t)stream, sm, codes, flags, tile_off, ovf, head_start, base3, base4, n_kv, bidx, S, S_pad, (u16*)out, out_head_stride, out_row_stride);
  return launch_status("gaac_decode_tiles");
}

}  // extern "C"
