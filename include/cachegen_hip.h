/*
 * cachegen_hip.h -- C ABI of the MI355X (gfx950) CacheGen KV codec library.
 *
 * Plain pointers and sizes only; every pointer named "device" must be memory the
 * GPU can access, `stream` is a hipStream_t passed as void* (NULL = the null
 * stream).  All functions are asynchronous with respect to the host, keep no
 * state between calls and return CG_OK or a negative CG_ERR_* code;
 * cg_last_error() then holds a message for the calling thread.
 *
 * The encode and decode entry points launch one block per (channel tile, row,
 * sub-chunk of 256 tokens) on a three-dimensional grid: at most 65535 rows
 * (layers, or 2 x layers for the *_kv functions) and 65535 sub-chunks per call,
 * CG_ERR_ARG beyond.
 *
 * Paths in the comments are relative to LMCache/ in the reference tree:
 *   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
 *   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
 *   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
 *   main.cpp   = third_party/torchac_cuda/main.cpp
 *   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
 *   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
 */
#ifndef CACHEGEN_HIP_H
#define CACHEGEN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CG_OK 0
#define CG_ERR_ARG (-1)      /* bad shape, stride, dtype or limit */
#define CG_ERR_LAUNCH (-2)   /* the HIP runtime refused a launch */
#define CG_ERR_WORKSPACE (-3)/* workspace too small */

#define CG_DT_F16 0
#define CG_DT_BF16 1

#define CG_MAX_TOKENS_PER_STREAM 256 /* cachegen_basics.py:8, enc_new.cu:9-15 */
#define CG_MAX_LP 129                /* table length limit of this library (reference: 48 / 64) */
#define CG_MAX_LEVELS 8              /* quantization levels one cg_encode_kv_levels call takes */

/* Message for the last error returned on this thread ("" if none). */
const char *cg_last_error(void);
/* ABI version of the library: bumped when a signature changes. */
int cg_abi_version(void);

/* ---------------------------------------------------------------------------
 * The four entry points of the reference's extension module (main.cpp:14-17).
 * Strides are in elements.  Tables are int16 bit patterns of uint16 values.
 * ------------------------------------------------------------------------- */

/* torchac_cuda.calculate_cdf (cal_cdf.cu:68-129).
 * sym  device int8  [nl, nt, nc], strides (s0, s1, s2), values in [0, max_bins)
 * cdf  device int16 [nl, nc, max_bins + 1], contiguous, written
 * Counters are 16 bits wide as in the reference, so nt <= 65535 is required. */
int cg_calculate_cdf(const int8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                     int64_t s0, int64_t s1, int64_t s2, int max_bins,
                     int16_t *cdf, void *stream);

/* torchac_cuda.encode_fast_new (enc_new.cu:355-451).
 * cdf      device int16 [nl, nc, lp] contiguous
 * sym      device int8  [nl, nt, nc], strides (s0, s1, s2), nt <= 256
 * out      device uint8 [nl, nc, cap], strides (o0, o1, 1); stream (l, c) is written
 *          to out[l, c, 0:length]; bytes past the length are left untouched
 * lengths  device int32 [nl, nc] contiguous, written.  A stream longer than `cap`
 *          is truncated to `cap` stored bytes while its full length is reported. */
int cg_encode_fast_new(const int16_t *cdf, int lp, const int8_t *sym,
                       int64_t nl, int64_t nt, int64_t nc,
                       int64_t s0, int64_t s1, int64_t s2,
                       uint8_t *out, int64_t cap, int64_t o0, int64_t o1,
                       int32_t *lengths, void *stream);

/* torchac_cuda.decode_fast_new (dec_new.cu:314-393): streams in a padded buffer.
 * padded   device uint8 [nl, nc, cap], strides (p0, p1, 1)
 * lengths  device int32 [nl, nc] contiguous (kept for the reference's signature: the
 *          decoder stops after nt symbols and does not need them)
 * out      device uint8 [nl, nt, nc], strides (o0, o1, o2), written */
int cg_decode_fast_new(const int16_t *cdf, int lp, const uint8_t *padded, int64_t cap,
                       int64_t p0, int64_t p1, const int32_t *lengths,
                       int64_t nl, int64_t nt, int64_t nc,
                       uint8_t *out, int64_t o0, int64_t o1, int64_t o2, void *stream);

/* torchac_cuda.decode_fast_prefsum (dec_new.cu:403-479): streams concatenated in
 * (layer, channel) order.
 * bytes    device uint8 [nbytes]; the decoder loads whole aligned 32-bit
 *          words, so up to 3 bytes on either side of the buffer (inside the same aligned
 *          words) are read but never used
 * prefix   device int64 [nl, nc] contiguous: INCLUSIVE running sum of the stream
 *          lengths (decoder.py:70); stream g = l*nc + c is bytes[prefix[g-1]:prefix[g]] */
int cg_decode_fast_prefsum(const int16_t *cdf, int lp, const uint8_t *bytes, int64_t nbytes,
                           const int64_t *prefix, int64_t nl, int64_t nt, int64_t nc,
                           uint8_t *out, int64_t o0, int64_t o1, int64_t o2, void *stream);

/* ---------------------------------------------------------------------------
 * Fused forms of the Python-side tensor code around those kernels.
 *
 * A KV cache is a 16-bit float tensor indexed (layer, k|v, token, head, dim) with
 * element strides (sl, skv, st, sh, 1): [L,2,T,H,D] ("vllm") and [L,2,H,T,D]
 * ("huggingface") are both expressible (encoder.py:341-342, decoder.py:169-173).
 * C = H*D channels; "2L" rows are the L key layers followed by the L value layers
 * (encoder.py:263).  Tokens are cut into chunks of `chunk_tokens` (one table per
 * chunk, layer and channel: one `to_bytes` call of the reference each) and every
 * chunk into sub-chunks of at most 256 tokens (encoder.py:279-292); sub-chunks
 * are numbered consecutively over the whole tensor (nsub of them).  A stream is
 * one (sub-chunk, row of 2L, channel), numbered in that order.
 * ------------------------------------------------------------------------- */

/* torch_quant_vectorized on K and V (encoder.py:42-59, 72-83, 258-263).
 * kv          device fp16/bf16 KV cache (kv_dt, strides above)
 * key_bins    device float32 [L], value_bins likewise (encoder.py:311-322)
 * sym         device uint8 [2L, T, C] contiguous, written
 * maxima      device 16-bit [2, L, T] contiguous in kv_dt, written: row maxima,
 *             maxima[0] = max_tensors_key, maxima[1] = max_tensors_value */
int cg_quantize_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                   int64_t sl, int64_t skv, int64_t st, int64_t sh,
                   const float *key_bins, const float *value_bins,
                   uint8_t *sym, void *maxima, void *stream);

/* Number of sub-chunks / chunks for T tokens cut every chunk_tokens. */
int64_t cg_num_chunks(int64_t T, int64_t chunk_tokens);
int64_t cg_num_subchunks(int64_t T, int64_t chunk_tokens);

/* Bytes of device workspace cg_encode_kv needs. */
size_t cg_encode_kv_workspace(int64_t L, int64_t T, int64_t C, int64_t chunk_tokens);

/* encode_function for every chunk at once (encoder.py:247-301), including
 * collect_bytes (encoder.py:209-222).
 * cdf         device int16 [nchunks, 2L, C, max_bins+1], written
 * maxima      device 16-bit [2, L, T] in kv_dt, written
 * lengths     device int32 [nsub, 2L, C], written: bytes of every stream
 * offsets     device int64 [nsub*2L*C + 1], written: exclusive running sum of the
 *             lengths; offsets[last] = total payload bytes
 * payload     device uint8 [payload_cap], written: all streams back to back in
 *             stream order; the streams of sub-chunk g are
 *             payload[offsets[g*2L*C] : offsets[(g+1)*2L*C]] = that sub-chunk's
 *             `bytestream` tensor.  payload_cap >= 256 * number of streams is
 *             always enough.
 * status      device int32 [1], written: 0, or 1 if a stream exceeded 256 bytes
 *             (the reference overruns its buffer there; here the stream is cut).
 * workspace   device scratch of cg_encode_kv_workspace(...) bytes, 256-aligned
 * delta_group 0 for the reference's codec.  > 0 (no counterpart in the reference): inside
 *             every sub-chunk, tokens form groups of this many; the first row of a group
 *             (the anchor) is quantized as is, every other row as its float32 difference
 *             from the anchor row, with the row maximum of the differences rounded to the
 *             16-bit format; cg_decode_kv with the same value adds the reconstructed
 *             anchor back. */
int cg_encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                 int64_t sl, int64_t skv, int64_t st, int64_t sh,
                 const float *key_bins, const float *value_bins, int max_bins,
                 int64_t chunk_tokens, int delta_group,
                 int16_t *cdf, void *maxima, int32_t *lengths, int64_t *offsets,
                 uint8_t *payload, int64_t payload_cap, int32_t *status,
                 void *workspace, size_t workspace_bytes, void *stream);

/* Test hook: cg_encode_kv with the internal choices that have two forms switched by `flags` to
 * the form the call would not take by itself.  Same arguments and the same results as
 * cg_encode_kv, which is what the tests that call it check.  No counterpart in the reference.
 * CG_TEST_BYTE_SYMBOLS          every row's symbols cross from the quantizer to the coder a byte a
 *                               symbol (cg_encode_kv packs rows of at most 15 symbols four bits a symbol)
 * CG_TEST_TABLES_IN_QUANTIZER   the quantizer counts the symbols and writes the tables, however few
 *                               chunks the call has (cg_encode_kv does so from 512 (row, chunk) pairs on,
 *                               where the tables of all channels fit the LDS of one block; calls with
 *                               fewer pairs and chunks of more than 256 tokens cut the chunks into parts)
 * CG_TEST_SPLIT_CHUNKS          with the form above: every chunk of more than 256 tokens is counted in
 *                               parts of 256 tokens by separate blocks, whose counters are summed in memory
 * CG_TEST_TABLES_IN_CODER       never: the coder (one table per sub-chunk) or a separate pass over
 *                               the symbols (longer chunks) builds the tables */
#define CG_TEST_BYTE_SYMBOLS 1
#define CG_TEST_TABLES_IN_QUANTIZER 2
#define CG_TEST_TABLES_IN_CODER 4
#define CG_TEST_SPLIT_CHUNKS 8
int cg_test_encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                      int64_t sl, int64_t skv, int64_t st, int64_t sh,
                      const float *key_bins, const float *value_bins, int max_bins,
                      int64_t chunk_tokens, int delta_group,
                      int16_t *cdf, void *maxima, int32_t *lengths, int64_t *offsets,
                      uint8_t *payload, int64_t payload_cap, int32_t *status,
                      void *workspace, size_t workspace_bytes, void *stream, int flags);

/* The same KV cache encoded at `nlevels` quantization levels from ONE read of the tensor: the
 * adaptive-streaming use of the reference, which pre-encodes every chunk at QUANT_LEVEL 1..3
 * by calling the serializer once per level (run_adaptation.py:63-72, src/utils.py:357-377).
 * Every row is loaded once and its maximum found once; its symbols are written once per level
 * and each level is then coded exactly as cg_encode_kv codes it, so level v's tables, lengths,
 * offsets and payload are byte-identical to a cg_encode_kv call with key_bins[v],
 * value_bins[v], max_bins[v].
 * key_bins, value_bins   HOST arrays of nlevels device pointers (float32 [L] each)
 * max_bins               HOST array of nlevels ints
 * cdf, lengths, offsets, payload   HOST arrays of nlevels device pointers, shaped as in
 *                        cg_encode_kv (cdf[v]: [nchunks, 2L, C, max_bins[v]+1]); payload_cap
 *                        a HOST array of nlevels capacities
 * maxima                 device 16-bit [2, L, T]: the row maxima do not depend on the level
 * status                 device int32 [nlevels]
 * workspace              cg_encode_kv_levels_workspace(...) bytes, 256-aligned
 * 1 <= nlevels <= CG_MAX_LEVELS.  Tensors whose head size or strides are not multiples of 8
 * are quantized once per level instead. */
size_t cg_encode_kv_levels_workspace(int64_t L, int64_t T, int64_t C, int64_t chunk_tokens, int nlevels);
int cg_encode_kv_levels(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                        int64_t sl, int64_t skv, int64_t st, int64_t sh,
                        int nlevels, const float *const *key_bins, const float *const *value_bins,
                        const int *max_bins, int64_t chunk_tokens,
                        int16_t *const *cdf, void *maxima, int32_t *const *lengths,
                        int64_t *const *offsets, uint8_t *const *payload, const int64_t *payload_cap,
                        int32_t *status, void *workspace, size_t workspace_bytes, void *stream);

/* Exclusive running sum of stream lengths: offsets[0] = 0, offsets[i+1] =
 * offsets[i] + lengths[i] (the inclusive sums of decoder.py:70 are offsets[1:]).
 * scratch: device, cg_scan_workspace(n) bytes. */
size_t cg_scan_workspace(int64_t n);
int cg_scan_lengths(const int32_t *lengths, int64_t n, int64_t *offsets,
                    void *scratch, size_t scratch_bytes, void *stream);

/* cg_scan_lengths for callers that cannot allocate device memory and have no workspace to
 * pass (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).
 * No counterpart in the reference.  Same results as cg_scan_lengths; the partial sums live
 * in an array that is part of the library's device image (about 64 KiB on every GPU the
 * library runs on, held until the process ends), so the call allocates and frees nothing.
 * n <= CG_SCAN_STATIC_MAX_LENGTHS, CG_ERR_WORKSPACE otherwise.  All calls on one GPU share that
 * array: two calls whose kernels overlap on the same GPU (different streams, or different
 * threads on different streams) race; calls queued on one stream do not.  The first call on a
 * device looks the array's address up (hipGetSymbolAddress) with that device current. */
#define CG_SCAN_STATIC_MAX_LENGTHS (16 * 1024 * 1024)
int cg_scan_lengths_static(const int32_t *lengths, int64_t n, int64_t *offsets, void *stream);

/* decode_function_gpu + do_dequantize + the final cast and layout (decoder.py:
 * 77-112, 24-34, 159-173) for every chunk at once.
 * cdf, maxima, offsets, payload: as written by cg_encode_kv (maxima in max_dt);
 *             whole aligned 32-bit words of the payload are loaded, see
 *             cg_decode_fast_prefsum
 * out         device fp16/bf16 KV cache (out_dt, strides (ol, okv, ot, oh, 1)), written.
 *             ot and oh must not be negative, and 256 token rows of one layer's keys or
 *             values must span less than 4 GiB (((H-1)*oh + D-1 + 255*ot) * 2 + 2 bytes):
 *             the kernel addresses them with a 32-bit offset from a per-block base;
 *             CG_ERR_ARG otherwise */
int cg_decode_kv(const int16_t *cdf, int max_bins, const void *maxima, int max_dt,
                 const int64_t *offsets, const uint8_t *payload, int64_t payload_bytes,
                 const float *key_bins, const float *value_bins,
                 int64_t L, int64_t T, int64_t H, int64_t D, int64_t chunk_tokens,
                 int delta_group,
                 void *out, int out_dt, int64_t ol, int64_t okv, int64_t ot, int64_t oh,
                 void *stream);

/* ---------------------------------------------------------------------------
 * Tables as histogram counts, for containers that store the counts (no counterpart in
 * the reference, whose container pickles the tables; the relation inverted here is
 * cal_cdf.cu:29-49).  A group is one (chunk, row): C channels sharing a token count
 * tokens[g] <= 256.
 * ------------------------------------------------------------------------- */

/* cdf     device int16 [ngroups, C, max_bins+1]
 * tokens  device int32 [ngroups]: tokens the tables of group g were built over (1..256)
 * counts  device uint8 [ngroups, C, max_bins], written: histogram counts, 256 stored as 255
 * nsym    device int32 [ngroups], written: 1 + the largest symbol that occurs in the group
 * inexact device int32 [1], written: 1 if some table is not the table of any histogram */
int cg_tables_to_counts(const int16_t *cdf, int max_bins, int64_t ngroups, int64_t C,
                        const int32_t *tokens, uint8_t *counts, int32_t *nsym, int32_t *inexact,
                        void *stream);

/* Ragged form of `counts`: out[starts[g] + ch*nsym[g] + j] = counts[g, ch, j], j < nsym[g]. */
int cg_pack_counts(const uint8_t *counts, int max_bins, int64_t ngroups, int64_t C,
                   const int32_t *nsym, const int64_t *starts, uint8_t *out, void *stream);

/* Ragged counts back to tables.
 * data    device uint8 [data_bytes]: as written by cg_pack_counts (never read outside)
 * nsym    device uint8 [ngroups]; starts device int64 [ngroups]
 * cdf     device int16 [ngroups, C, max_bins+1], written
 * invalid device int32 [1], written: 1 if some channel's counts do not add up to tokens[g] */
int cg_counts_to_tables(const uint8_t *data, int64_t data_bytes, int max_bins, int64_t ngroups, int64_t C,
                        const int32_t *tokens, const uint8_t *nsym, const int64_t *starts, int16_t *cdf,
                        int32_t *invalid, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CACHEGEN_HIP_H */
