/* C-ABI of libgaac_hip.so: the MI355X (gfx950) kernels behind gaac_amd.{codec,encoder,kernel,kv_cache,paged}.
 *
 * Conventions for every entry point:
 *   - all pointers are DEVICE pointers (plain, no framework types); `stream` is a hipStream_t passed as void*;
 *   - nothing is allocated, nothing synchronizes, all work is enqueued on `stream` (graph-capture safe);
 *   - returns 0 on success, -1 for rejected arguments, a positive hipError_t for a failed launch; the message
 *     of the last failure on the calling thread is returned by gaac_last_error().
 *   - BF16 tensors are passed as void* (16-bit patterns); `kind` is 0 for K, 1 for V.
 *
 * Byte order inside a 16-token tile (sign/mantissa and code bytes) is the gfx950 MFMA operand order documented in
 * gaac_amd/csrc/gaac_core.h.  K tag words and K escape bytes have the reference's order (one tag word per token; escapes by
 * token, then group).  V tag words and V escape bytes are transposed within the tile: tag word a of a tile belongs to GROUP a
 * and holds the tags of its 16 tokens (token j at bits 2j), and the tile's escape bytes run by group, then token.  Per-tile
 * escape byte counts, tile offsets and head starts are the reference's numbers.
 * Citations are to the reference interface each entry point replaces.
 */
#ifndef GAAC_HIP_H
#define GAAC_HIP_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* gaac_last_error(void);

/* exponent_hist(x, n_kv), /root/reference/gaac/codec.py:80-84.  x: bf16 [n_tokens, n_kv, 128] token-major;
 * hist: int64 [n_kv*128, 256], ACCUMULATED into (zero it first). */
int gaac_exponent_hist(const void* x, long n_tokens, int n_kv, long long* hist, void* stream);

/* bases_from_hist(hist, n_kv), /root/reference/gaac/codec.py:70-77.  rows = n_kv*128; base3/base4: uint8 [rows]. */
int gaac_bases_from_hist(const long long* hist, int rows, uint8_t* base3, uint8_t* base4, void* stream);

/* TileEncoder.encode_tiles, /root/reference/gaac/encoder.py:16-66, 94-102 (same math as Codec.encode, codec.py:133-184).
 * x: bf16, element (h, s, c) at x[h*x_head_stride + s*x_row_stride + c] (head-major [H, S_in, 128] or a token-major prompt
 * [S_in, H, 128] without a transposing copy; rows 16-byte aligned); tiles 0..ceil(S/16)-1 of every head are written to
 * sm [H, S_pad*128], codes [H, S_pad*48], flags [H, S_pad]; escape bytes of tile (h, t) go to esc_slots[(h*ntiles+t)*1280 ...];
 * tile_bytes: int32 [H, ntiles].  Head h uses base row bidx[h] (bidx != NULL) or h % n_kv. */
int gaac_encode_tiles(int kind, const void* x, long x_head_stride, long x_row_stride, int H, int S, int S_pad, const uint8_t* base3,
                      const uint8_t* base4, int n_kv, const int* bidx, uint8_t* sm, uint8_t* codes, int* flags, uint8_t* esc_slots,
                      int* tile_bytes, void* stream);

/* TileEncoder.compact, /root/reference/gaac/encoder.py:69-76, 104-109: writes tile_off[h, t] = sum of tile_bytes[h, 0..t) (int32
 * [H, ntiles], output) and copies tile (h, t)'s tile_bytes[h, t] escape bytes from its 1280-byte slot to
 * ovf + head_start[h] + tile_off[h, t]. */
int gaac_compact(const uint8_t* esc_slots, const int* tile_bytes, int* tile_off, const int* head_start, uint8_t* ovf,
                 int H, int ntiles, void* stream);

/* row_offsets(flags, S), /root/reference/gaac/codec.py:221-225.  flags: int32 [H, S_pad]; out: int32 [H, S];
 * chunk_sums: scratch, int32 [H * ceil(S / 2048)] (escape bytes per chunk of 2048 rows; written, then read). */
int gaac_row_offsets(const int* flags, int H, int S, int S_pad, int* chunk_sums, int* out, void* stream);

/* Codec.decode, /root/reference/gaac/codec.py:186-218.  Page fields as in the reference's Page dataclass
 * (codec.py:87-102) with tile_off [H, S_pad/16]; out: bf16, element (h, s, c) at out[h*out_head_stride + s*out_row_stride + c]. */
int gaac_decode_tiles(int kind, const uint8_t* sm, const uint8_t* codes, const int* flags, const int* tile_off, const uint8_t* ovf,
                      const int* head_start, const uint8_t* base3, const uint8_t* base4, int n_kv, const int* bidx, int H, int S,
                      int S_pad, void* out, long out_head_stride, long out_row_stride, void* stream);

/* gaac_attn_launch, /root/reference/gaac/kernel.py:296-326 (kernels :48-294).  Same 16 store tensors, q [B*n_q, 128] bf16,
 * slot map [B] (slot < 0 = padded row, output 0; NULL = the identity, row b attends over cache heads b*n_kv ..), SL [cache heads] compressed tokens per head, S_pad = token stride of a
 * head, nsplit, and the optional raw tail kt/vt [cache heads, TCAP, 128] bf16 with lengths TL (kt == NULL: no tail).
 * NB = rows of the base tables (n_kv, or the number of cache heads for per-sequence bases).
 * Differences from the reference entry: the caller passes the partial buffers pm, pl [B*n_q*NSLOT] and
 * pa [B*n_q*NSLOT*128] (fp32, NSLOT = nsplit; the tail is folded into the last split's partial) and `out` [B*n_q, 128] bf16 instead of having them
 * allocated inside; GQA group sizes 1..16 are accepted (reference: 1..8). */
int gaac_attn_launch(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP,
    float* pm, float* pl, float* pa, void* out, void* stream);

/* The two halves of gaac_attn_launch on their own (the split pass = gaac_attn + gaac_tail of kernel.py:48-279, the merge =
 * gaac_combine of kernel.py:281-294), for callers that time or schedule them separately.  n_rows = B*n_q. */
int gaac_attn_split(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, float* pm, float* pl, float* pa, void* stream);
int gaac_attn_combine(const float* pm, const float* pl, const float* pa, void* out, int n_rows, int nslot, void* stream);

/* gaac_attn_launch as ONE kernel: the merge of the NSLOT partials (gaac_combine, kernel.py:281-294) is done inside the split kernel
 * by the last (up to sixteen) blocks of each (batch row, kv head) in index order, each taking a share of the head's output, without
 * atomics.  epoch[0] holds the epoch of the last merged launch; this launch's epoch is that + 1.  Partials travel as 64-bit records
 * (fp32 bits | epoch << 32) written and read with single 64-bit accesses, so a merging block recognises the records of this launch
 * without waiting for an acknowledgement; it re-reads records that have not arrived yet.  Every block stores the epoch it works
 * under into its arrival mark epoch[2 + block] when its first wave is through its tiles; the last block of the grid stores the new
 * epoch as its last action, after it has seen the marks of all blocks (so every block has read the word).  Every wait is bounded (about 0.1 s): instead of hanging, a launch ORs failure bits into epoch[1]: 1 = a merging block gave
 * up waiting for a partial and wrote its rows as NaN, 2 = the last block gave up waiting for the other blocks and left epoch[0]
 * alone.  Poll epoch[1] where the caller polls its other device-side error words.
 * pm, pl: records [B*n_q*nsplit]; pa: records [B*n_q*nsplit*128]; epoch: uint32 [2 + B*n_kv*nsplit] (epoch word, failure bits, one
 * arrival mark per block of the launch).  Zero epoch, pm, pl and pa before the first
 * launch and to re-arm them after a failed launch.  Launches of any shape may share them (buffers sized for the largest) as long as
 * they are ordered on one stream.  The fp32 partial buffers of gaac_attn_split / gaac_attn_launch must be other memory than these
 * records (plain values could be taken for records of some epoch).
 * S_all >= 0: every cache head the launch addresses holds exactly S_all compressed tokens (a Page: lengths are known to the host);
 * SL is then not read and may be NULL, which takes one dependent load off the start of every block.  S_all < 0: lengths come from SL. */
int gaac_attn_fused(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, int S_all,
    unsigned long long* pm, unsigned long long* pl, unsigned long long* pa, unsigned int* epoch, void* out, void* stream);

/* gaac_attn_fused for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses that forbid it): the
 * same launch, but the partial records and the epoch words live in a 4 MiB array built into the library (one copy per GPU, held from
 * load to process end) instead of caller memory; the call itself allocates nothing.  It has no counterpart in the reference, whose
 * entry allocates its partials on every call (kernel.py:306-307).  Limit: B*n_q*nsplit <= 4000 partial rows (the headline launch uses
 * 1024); larger launches are rejected with -1 and a message.  All calls on one GPU share the array: they must be ordered on one
 * stream (calls that overlap on a GPU race), and nothing needs clearing between them (the epoch tells launches apart).  The array
 * of the stream's device is used (the calling thread's current device for the null stream); that device must be the calling
 * thread's current one when its array is first touched.  The first touch is a runtime query that cannot run while a stream is
 * capturing: call gaac_static_init() (no arguments, current device, any time before the capture), or make one call outside the
 * capture; a first call from inside a capture is rejected with a message.
 * gaac_static_flags copies the array's failure bits (epoch[1] of gaac_attn_fused) to *flags_out (device memory) on the stream;
 * gaac_static_reset re-arms the array after a failed launch (epoch words and records to zero, by a kernel, so it can be captured). */
int gaac_static_init(void);
int gaac_static_reset(void* stream);
int gaac_static_flags(unsigned int* flags_out, void* stream);
int gaac_attn_fused_static(
    const uint8_t* smk, const uint8_t* ck, const int* fk, const int* tok, const uint8_t* ovk, const int* ohsk, const uint8_t* b3k, const uint8_t* b4k,
    const uint8_t* smv, const uint8_t* cv, const int* fv, const int* tov, const uint8_t* ovv, const int* ohsv, const uint8_t* b3v, const uint8_t* b4v,
    const void* q, const int* slot, int B, int n_q, int n_kv, const int* SL, int S_pad, float scale, int nsplit, int NB,
    const void* kt, const void* vt, const int* TL, int TCAP, int S_all, void* out, void* stream);

/* CompressedKVCache.append, /root/reference/gaac/kv_cache.py:172-181 (kernels _append_one/_append_kv/_advance, :22-96), as one
 * launch: row i = b*n_kv + kvh of k_new/v_new [B, n_kv, 128] bf16 goes to tail row tail_len[h] of cache head
 * h = slots[b]*n_kv + kvh (slots[b] < 0: skipped); when that fills the 16-row tail the tile is compressed in place as tile S[h]/16
 * (token stride cap), its escape bytes are appended at ovf + h*ovf_cap + ovf_used[h], and tile_off, ovf_used, tail_len and S advance.
 * Per kind: tail bf16 [H,16,128], base3/base4 u8 [NB,128] (row h % NB), sm u8 [H,cap*128], codes u8 [H,cap*48], flags i32 [H,cap],
 * ovf u8 [H*ovf_cap], tile_off i32 [H,cap/16], ovf_used i32 [H].  Instead of writing out of bounds the kernel ORs into *err:
 * 1 = a head was at capacity (token dropped), 2 = an escape stream was full (tile stored with zero tags). */
int gaac_cache_append(
    const int* slots, int B, int n_kv, const void* k_new, const void* v_new, int* tail_len, int* S, int cap, int ovf_cap, int NB,
    void* k_tail, const uint8_t* k_base3, const uint8_t* k_base4, uint8_t* k_sm, uint8_t* k_codes, int* k_flags, uint8_t* k_ovf, int* k_tile_off, int* k_ovf_used,
    void* v_tail, const uint8_t* v_base3, const uint8_t* v_base4, uint8_t* v_sm, uint8_t* v_codes, int* v_flags, uint8_t* v_ovf, int* v_tile_off, int* v_ovf_used,
    int* err, void* stream);

/* ---- paged slot pool (the layout of /root/reference/gaac/vllm/paged_kernel.py:3-6 and store.py:17-19) -------------------------------
 * pool: tile slots of TS bytes, physical tile p = block*2*n_kv + 2*kvh + kind: [0,2048) sign/mantissa | [2048,2816) codes |
 * [2816,2880) 16 tag words | [2880,TS) escape bytes.  mt int32 [num_blocks*2*n_kv]: p = compressed in its slot, ~r = raw BF16 tile r of
 * raw [tiles][16][128].  stack/top: free raw tiles; err: failed pops.  Bases uint8 [n_kv,128].  TS >= 2896 (a slot with no room for
 * escape bytes would hold no tile the raw pool could not).  No kernel reads or writes outside the slots. */

/* LayerState.store -> _store_tiles, store.py:22-105.  key/value: bf16 rows [num_tokens][n_kv][128] with row strides in elements;
 * ent int32 [n_ent][4] = (block, first token row, offset in block, rows), block < 0 = inactive; freeq int32 [n_ent*2*n_kv] receives
 * the raw tiles to give back (-1 = none); call gaac_paged_free on it afterwards (pops and pushes never share a launch). */
int gaac_paged_store(const void* key, const void* value, long k_stride, long v_stride, const int* ent, int n_ent,
                     uint8_t* pool, int TS, void* raw, int* mt, int* stack, int* top, int* err, int* freeq,
                     const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int n_kv, void* stream);
/* _free_tiles, store.py:108-114. */
int gaac_paged_free(const int* freeq, int n_items, int* stack, int* top, void* stream);
/* LayerState.release_blocks -> _release_blocks, store.py:164-174: raw tiles of dead blocks go back, their mode entries are reset. */
int gaac_paged_release(const int* blocks, int n_blocks, int* mt, int* stack, int* top, int n_kv, void* stream);
/* LayerState.decode_blocks -> _decode_tiles, store.py:117-161: pairs int32 [n_pairs][3] = (block, first output row, valid rows <= 16);
 * sk/sv: bf16 [rows][n_kv][128] with row stride row_stride elements. */
int gaac_paged_decode(const uint8_t* pool, int TS, const void* raw, const int* mt, const int* pairs, int n_pairs, void* sk, void* sv,
                      long row_stride, const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int n_kv, void* stream);
/* paged_attention -> gaac_vpaged_launch, paged_kernel.py:42-277: decode attention of B rows over the pool through the block table
 * bt int32 [B][bt_stride] and the mode table; seq_lens int32 [B] (tokens incl. the filling block; no separate tail); max_seq_len =
 * an upper bound of seq_lens known to the host (checked against the block table's width).  Any nsplit >= 1 works for any length (a
 * block resolves 1024 tiles of its split at a time).  Partial records pm, pl [B*n_q*nsplit], pa [B*n_q*nsplit*128] and the epoch
 * buffer [2 + B*n_kv*nsplit] as in gaac_attn_fused; out bf16 [B*n_q][128].
 * freeq != NULL: the launch also does the work of gaac_paged_free(freeq, n_free, stack, top) for the queue the preceding
 * gaac_paged_store filled (the attention pops nothing, so pushes cannot race a pop here): a decode step is then two launches
 * instead of the reference's three (store.py:108-114 is a launch of its own). */
int gaac_paged_attn(const uint8_t* pool, int TS, const void* raw, const int* mt, const int* bt, int bt_stride, const int* seq_lens,
                    int max_seq_len, const void* q, int B, int n_q, int n_kv, float scale, int nsplit,
                    const uint8_t* b3k, const uint8_t* b4k, const uint8_t* b3v, const uint8_t* b4v, int NB,
                    unsigned long long* pm, unsigned long long* pl, unsigned long long* pa, unsigned int* epoch, void* out,
                    const int* freeq, int n_free, int* stack, int* top, void* stream);

/* Baseline, not part of the compressed path: decode attention over UNCOMPRESSED bf16 K/V [B*n_kv][head_stride_tokens][128] (S tokens
 * per head, or seq_lens[b] <= S tokens for batch row b when seq_lens != NULL) with the same block / wave / MFMA structure, merge and
 * partial buffers as gaac_attn_fused.  The reference compares against flash-attn (examples/attention.py:29-30); this is the same-GPU
 * counterpart for that comparison. */
int gaac_bf16_attn(const void* k, const void* v, int S, const int* seq_lens, long head_stride_tokens, const void* q, int B, int n_q,
                   int n_kv, float scale, int nsplit, unsigned long long* pm, unsigned long long* pl, unsigned long long* pa,
                   unsigned int* epoch, void* out, void* stream);

#ifdef __cplusplus
}
#endif
#endif
