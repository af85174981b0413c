// CacheGen KV codec for MI355X (gfx950): hand-written HIP kernels behind a C ABI.
//
// The codec is HBM/ALU-bound integer work with no dense contraction, so there is
// no MFMA here.  The mapping everywhere is one lane = one (row, channel) stream
// and one wavefront = 64 adjacent channels of one row, which keeps every symbol
// and KV access of a wave on one contiguous segment; per-block tables live in LDS
// as 16-bit entries, one row of lanes per table entry (every lane has a column of its
// own; lanes whose symbols differ still meet on LDS banks now and then, which measured
// at 40 to 60 % of the LDS-busy cycles and does not limit these kernels: they are bound
// by vector instruction issue).  This file is the one translation unit: it includes the
// kernels and the launch helpers and defines the C ABI.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#include <hip/hip_runtime.h>

#include <climits>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <atomic>
#include <mutex>

#include "cachegen_hip.h"

// The float32 steps of quantisation and dequantisation are rounded one by one, as eager
// tensor code rounds them: no fused multiply-add anywhere in this file.
#pragma clang fp contract(off)


#include "common.hpp"
#include "quantize.hpp"
#include "tables.hpp"
#include "quantize_tables.hpp"
#include "encoder.hpp"
#include "decoder.hpp"
#include "scan_compact.hpp"
#include "launch.hpp"
#include "tables_wire.hpp"

// ======================================================================================
// Scratch of the entry point that allocates nothing (cg_scan_lengths_static): the partial sums
// of the multi-block running sum, one int64 per 2048 lengths plus one.  Every GPU the library
// runs on holds its own copy of this array, at its own address, until the process ends.  In host
// code the array's name is only a handle for hipGetSymbolAddress: kernels and copies get the
// device address looked up once per device below, never the name.
// ======================================================================================
constexpr int64_t kStaticScanMaxLengths = CG_SCAN_STATIC_MAX_LENGTHS;
constexpr size_t kStaticScanBytes = (size_t)(kStaticScanMaxLengths / kScanTile + 2) * sizeof(int64_t);
static __device__ __align__(256) unsigned char scratch[kStaticScanBytes];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_static_scratch_mutex;
void *g_static_scratch[kMaxDevices];          // device address of `scratch` on each GPU, once looked up

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void **ptr)
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(CG_ERR_LAUNCH, "scan_lengths_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(CG_ERR_ARG, "scan_lengths_static: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (!g_static_scratch[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return fail(CG_ERR_LAUNCH, "scan_lengths_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_static_scratch[dev] = p;
    }
    *ptr = g_static_scratch[dev];
    return CG_OK;
}

}  // namespace

// ======================================================================================
// C ABI
// ======================================================================================
extern "C" {

const char *cg_last_error(void) { return g_error; }
int cg_abi_version(void) { return 5; }

int64_t cg_num_chunks(int64_t T, int64_t chunk_tokens)
{
    if (T <= 0 || chunk_tokens <= 0) return 0;
    return ceil_div(T, chunk_tokens);
}

int64_t cg_num_subchunks(int64_t T, int64_t chunk_tokens)
{
    if (T <= 0 || chunk_tokens <= 0) return 0;
    const int64_t nchunks = ceil_div(T, chunk_tokens);
    const int64_t last = T - (nchunks - 1) * chunk_tokens;
    return (nchunks - 1) * ceil_div(chunk_tokens, kSub) + ceil_div(last, kSub);
}

int cg_calculate_cdf(const int8_t *sym, int64_t nl, int64_t nt, int64_t nc, int64_t s0, int64_t s1,
                     int64_t s2, int max_bins, int16_t *cdf, void *stream)
{
    if (!sym || !cdf) return fail(CG_ERR_ARG, "calculate_cdf: null pointer");
    if (nl <= 0 || nt <= 0 || nc <= 0) return fail(CG_ERR_ARG, "calculate_cdf: empty input");
    if (max_bins < 1 || max_bins + 1 > CG_MAX_LP) return fail(CG_ERR_ARG, "Max bins must be less than %d", CG_MAX_LP);
    if (nt > 65535) return fail(CG_ERR_ARG, "calculate_cdf: at most 65535 tokens per table (16-bit counters)");
    return launch_cdf(reinterpret_cast<const uint8_t *>(sym), nullptr, 0, nl, nt, nc, s0, s1, s2, max_bins, nt,
                      reinterpret_cast<uint16_t *>(cdf), static_cast<hipStream_t>(stream));
}

int cg_encode_fast_new(const int16_t *cdf, int lp, const int8_t *sym, int64_t nl, int64_t nt, int64_t nc,
                       int64_t s0, int64_t s1, int64_t s2, uint8_t *out, int64_t cap, int64_t o0,
                       int64_t o1, int32_t *lengths, void *stream)
{
    if (!cdf || (!sym && nt > 0) || !out || !lengths) return fail(CG_ERR_ARG, "encode: null pointer");
    if (int rc = check_lp(lp, "encode")) return rc;
    if (nl <= 0 || nc <= 0 || nt < 0) return fail(CG_ERR_ARG, "encode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    if (cap <= 0 || cap > INT_MAX) return fail(CG_ERR_ARG, "encode: bad output buffer length");
    const int block = pick_block(nc, lp);
    EncodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<uint16_t *>(const_cast<int16_t *>(cdf));      // only read here
    a.lp = lp;
    a.sym = reinterpret_cast<const uint8_t *>(sym);
    a.s0 = s0;
    a.s1 = s1;
    a.s2 = s2;
    a.out = out;
    a.o0 = o0;
    a.o1 = o1;
    a.cap = (int32_t)cap;
    a.lengths = lengths;
    a.status = nullptr;
    int64_t nblocks;
    // nt == 0 still writes the two closing bits of every stream
    if (int rc = make_grid(nl, nc, nt ? nt : 1, nt ? nt : 1, 1, block, a.sg, nblocks)) return rc;
    if (nt == 0) a.sg.g.T = 0;
    const size_t shmem = (size_t)lp * (block + 2) * sizeof(uint16_t);      // TableStride<BS>::k16 per entry
    const bool aligned = aligned_to(out, 4) && o0 % 4 == 0 && o1 % 4 == 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid = stream_grid(a.sg, nblocks), blk(block);
    if (aligned) CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, false, false, false><<<grid, blk, shmem, st>>>(a)));
    else CG_DISPATCH_BS(block, (encode_streams_kernel<BS, false, false, false, false><<<grid, blk, shmem, st>>>(a)));
    return check_launch("encode");
}

int cg_decode_fast_new(const int16_t *cdf, int lp, const uint8_t *padded, int64_t cap, int64_t p0,
                       int64_t p1, const int32_t *lengths, int64_t nl, int64_t nt, int64_t nc,
                       uint8_t *out, int64_t o0, int64_t o1, int64_t o2, void *stream)
{
    if (!cdf || !padded || !lengths || !out) return fail(CG_ERR_ARG, "decode: null pointer");
    if (int rc = check_lp(lp, "decode")) return rc;
    if (nl <= 0 || nc <= 0 || nt <= 0) return fail(CG_ERR_ARG, "decode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    if (cap <= 0 || cap > INT_MAX) return fail(CG_ERR_ARG, "decode: bad padded buffer length");
    const int block = pick_block(nc, lp);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = lp;
    if (int rc = set_byte_window(a, padded, (nl - 1) * p0 + (nc - 1) * p1 + cap, "decode")) return rc;
    a.p0 = p0;
    a.p1 = p1;
    a.out_sym = out;
    a.o0 = o0;
    a.o1 = o1;
    a.o2 = o2;
    a.last_round_first = 0xFFFFFFFFu;     // one sub-chunk: a single round of blocks
    int64_t nblocks;
    if (int rc = make_grid(nl, nc, nt, nt, 1, block, a.sg, nblocks)) return rc;
    return launch_decode_symbols<SRC_PADDED>(a, nblocks, block, static_cast<hipStream_t>(stream));
}

int cg_decode_fast_prefsum(const int16_t *cdf, int lp, const uint8_t *bytes, int64_t nbytes,
                           const int64_t *prefix, int64_t nl, int64_t nt, int64_t nc, uint8_t *out,
                           int64_t o0, int64_t o1, int64_t o2, void *stream)
{
    if (!cdf || !prefix || !out || !bytes) return fail(CG_ERR_ARG, "decode: null pointer");
    if (int rc = check_lp(lp, "decode")) return rc;
    if (nl <= 0 || nc <= 0 || nt <= 0) return fail(CG_ERR_ARG, "decode: empty input");
    if (nt > kSub) return fail(CG_ERR_ARG, "Number of tokens should be less than or equal to %d", kSub);
    const int block = pick_block(nc, lp);
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = lp;
    if (int rc = set_byte_window(a, bytes, nbytes, "decode")) return rc;
    a.offsets = prefix;
    a.out_sym = out;
    a.o0 = o0;
    a.o1 = o1;
    a.o2 = o2;
    a.last_round_first = 0xFFFFFFFFu;     // one sub-chunk: a single round of blocks
    int64_t nblocks;
    if (int rc = make_grid(nl, nc, nt, nt, 1, block, a.sg, nblocks)) return rc;
    return launch_decode_symbols<SRC_PREFIX>(a, nblocks, block, static_cast<hipStream_t>(stream));
}

int cg_quantize_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                   int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
                   uint8_t *sym, void *maxima, void *stream)
{
    if (!kv || !key_bins || !value_bins || !sym || !maxima) return fail(CG_ERR_ARG, "quantize: null pointer");
    if (int rc = check_dt(kv_dt, "quantize")) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0) return fail(CG_ERR_ARG, "quantize: empty input");
    return launch_quantize(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, sym, maxima,
                           static_cast<hipStream_t>(stream));
}

size_t cg_scan_workspace(int64_t n) { return align_up((size_t)(ceil_div(n > 0 ? n : 1, kScanTile) + 1) * sizeof(int64_t), 256); }

int cg_scan_lengths(const int32_t *lengths, int64_t n, int64_t *offsets, void *scratch,
                    size_t scratch_bytes, void *stream)
{
    if (!lengths || !offsets || !scratch) return fail(CG_ERR_ARG, "scan: null pointer");
    if (n <= 0) return fail(CG_ERR_ARG, "scan: empty input");
    if (scratch_bytes < cg_scan_workspace(n)) return fail(CG_ERR_WORKSPACE, "scan: scratch too small");
    return launch_scan(lengths, n, INT_MAX, offsets, scratch, static_cast<hipStream_t>(stream));
}

int cg_scan_lengths_static(const int32_t *lengths, int64_t n, int64_t *offsets, void *stream)
{
    if (!lengths || !offsets) return fail(CG_ERR_ARG, "scan_lengths_static: null pointer");
    if (n <= 0) return fail(CG_ERR_ARG, "scan_lengths_static: empty input");
    if (n > kStaticScanMaxLengths)
        return fail(CG_ERR_WORKSPACE, "scan_lengths_static: %lld lengths exceed the built-in scratch (at most %lld); "
                                      "use cg_scan_lengths with a workspace", (long long)n, (long long)kStaticScanMaxLengths);
    void *ptr = nullptr;
    if (int rc = static_scratch(&ptr)) return rc;
    // every partial sum the second and third kernel read is written by the first kernel of this
    // same call, so nothing of the previous call's contents has to be cleared
    return launch_scan(lengths, n, INT_MAX, offsets, ptr, static_cast<hipStream_t>(stream));
}

}  // extern "C"

namespace {

// Workspace of the fused encoder, carved in this order: `nlevels` symbol areas (a 256-token
// slot per stream each), the coder's scratch tiles, and the small arrays of the two running sums.
struct EncodeWorkspace {
    size_t symbols_bytes;       // one level's symbols
    uint8_t *symbols, *scratch;
    void *scan_scratch, *tile_scan_scratch;
    int32_t *tile_sums, *group_sums;
    int64_t *tile_base;
    int64_t nsub, nstreams, ntiles;
    size_t total;

    EncodeWorkspace(void *base, int64_t L, int64_t T, int64_t C, int64_t chunk_tokens, int nlevels)
    {
        nsub = cg_num_subchunks(T, chunk_tokens);
        nstreams = nsub * 2 * L * C;
        ntiles = ceil_div(nstreams, kSlotTile);
        symbols_bytes = align_up((size_t)nstreams * kSub, 256);
        uint8_t *ws = static_cast<uint8_t *>(base);
        symbols = ws;
        ws += symbols_bytes * (size_t)nlevels;
        scratch = ws;           // kStreamCap bytes per stream, in tiles of kSlotTile word-interleaved streams
        ws += (size_t)ntiles * kSlotTile * kStreamCap;
        scan_scratch = ws;
        ws += cg_scan_workspace(nstreams);
        tile_sums = reinterpret_cast<int32_t *>(ws);           // bytes per tile of streams
        ws += align_up((size_t)ntiles * sizeof(int32_t), 256);
        tile_base = reinterpret_cast<int64_t *>(ws);           // their running sums
        ws += align_up((size_t)(ntiles + 1) * sizeof(int64_t), 256);
        tile_scan_scratch = ws;
        ws += cg_scan_workspace(ntiles);
        group_sums = reinterpret_cast<int32_t *>(ws);          // bytes per group of kTileGroup tiles
        ws += align_up((size_t)kMaxTileGroups * sizeof(int32_t), 256);
        total = (size_t)(ws - static_cast<uint8_t *>(base));
    }
};

}  // namespace

extern "C" {

size_t cg_encode_kv_workspace(int64_t L, int64_t T, int64_t C, int64_t chunk_tokens)
{
    return EncodeWorkspace(nullptr, L, T, C, chunk_tokens, 1).total;
}

size_t cg_encode_kv_levels_workspace(int64_t L, int64_t T, int64_t C, int64_t chunk_tokens, int nlevels)
{
    if (nlevels < 1 || nlevels > CG_MAX_LEVELS) return 0;
    return EncodeWorkspace(nullptr, L, T, C, chunk_tokens, nlevels).total;
}

}  // extern "C"

namespace {

// What one quantization level's outputs are.
struct LevelOut {
    const float *key_bins, *value_bins;
    int max_bins;
    int16_t *cdf;
    int32_t *lengths;
    int64_t *offsets;
    uint8_t *payload;
    int64_t payload_cap;
    int32_t *status;
};

// Tables, streams and payload of one level from its symbols (packed words `sym4`, or byte
// symbols [2L, T, C]): calculate_cdf + encode_fast_new + collect_bytes for every chunk
// (encoder.py:265-292, 209-222).
// The level's status word has been set to zero by an earlier launch of the same call.
// maxima, max_dt: the row maxima (packed symbols only); nibbles: the quantizer packed the rows
// of at most 15 symbols four bits a symbol (see narrow_alphabet).
// tables_ready: the tables were written by an earlier launch of the call (quantize_tables_kernel),
// which also set the workspace's group sums to zero.
int code_and_compact(const LevelOut &o, const uint32_t *sym4, const uint8_t *sym_bytes, const EncodeWorkspace &w,
                     int64_t L, int64_t T, int64_t C, int64_t chunk_tokens, hipStream_t s,
                     const void *maxima = nullptr, int max_dt = 0, bool nibbles = false, bool tables_ready = false)
{
    const int64_t rows = 2 * L;
    const int lp = o.max_bins + 1;
    uint16_t *tables = reinterpret_cast<uint16_t *>(o.cdf);

    const int block = pick_block(C, lp);
    EncodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = tables;
    a.lp = lp;
    a.nsub = w.nsub;
    a.out = w.scratch;
    a.cap = kStreamCap;
    a.lengths = o.lengths;
    a.status = o.status;
    a.key_bins = o.key_bins;
    a.value_bins = o.value_bins;
    a.L = L;
    int64_t nblocks;
    if (int rc = make_grid(rows, C, T, chunk_tokens, w.nsub, block, a.sg, nblocks)) return rc;
    const size_t shmem = (size_t)lp * (block + 2) * sizeof(uint16_t);      // TableStride<BS>::k16 per entry
    const dim3 grid = stream_grid(a.sg, nblocks), blk(block);
    // when every encoder block is exactly one tile of the scratch, the blocks leave their byte
    // counts behind and the compaction computes the stream offsets itself
    const bool fused_scan = block == kSlotTile && C % kSlotTile == 0;
    a.tile_sums = fused_scan ? w.tile_sums : nullptr;
    // few enough tiles: no scan launch either, the coder's blocks add the counts up by groups of
    // tiles (the sums were cleared by the quantizer that made the tables) and the compaction adds
    // up what lies before each tile
    const bool grouped = fused_scan && tables_ready && ceil_div(w.ntiles, kTileGroup) <= kMaxTileGroups;
    a.group_sums = grouped ? w.group_sums : nullptr;

    if (sym4) {
        // four tokens per word, read by one lane per channel
        a.sym4 = sym4;
        a.nibbles = nibbles ? 1 : 0;
        a.maxima = static_cast<const uint16_t *>(maxima);
        a.max_dt = max_dt;
        if (tables_ready) {
            if (fused_scan) encode_streams_kernel<kSlotTile, true, true, false, true, true><<<grid, blk, shmem, s>>>(a);
            else CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, true, false, true><<<grid, blk, shmem, s>>>(a)));
        } else if (chunk_tokens <= kSub) {
            // one sub-chunk per chunk: the encoder builds the tables itself
            if (fused_scan) encode_streams_kernel<kSlotTile, true, true, true, true, true><<<grid, blk, shmem, s>>>(a);
            else CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, true, true, true><<<grid, blk, shmem, s>>>(a)));
        } else {
            if (int rc = launch_cdf(nullptr, sym4, w.nsub, rows, T, C, 0, 0, 0, o.max_bins, chunk_tokens, tables, s,
                                    nibbles ? o.key_bins : nullptr, nibbles ? o.value_bins : nullptr)) return rc;
            if (fused_scan) encode_streams_kernel<kSlotTile, true, true, false, true, true><<<grid, blk, shmem, s>>>(a);
            else CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, true, false, true><<<grid, blk, shmem, s>>>(a)));
        }
    } else {
        // any shape or alignment: byte symbols [2L, T, C]
        if (int rc = launch_cdf(sym_bytes, nullptr, 0, rows, T, C, T * C, C, 1, o.max_bins, chunk_tokens, tables, s)) return rc;
        a.sym = sym_bytes;
        a.s0 = T * C;
        a.s1 = C;
        a.s2 = 1;
        CG_DISPATCH_BS(block, (encode_streams_kernel<BS, true, false, false, true><<<grid, blk, shmem, s>>>(a)));
    }
    if (int rc = check_launch("encode_kv")) return rc;

    const int64_t cblocks = ceil_div(w.nstreams, kCompactStreams);
    if (cblocks > INT_MAX) return fail(CG_ERR_ARG, "encode_kv: too many streams");
    const int32_t skew = (int32_t)(reinterpret_cast<uintptr_t>(o.payload) & 3u);
    if (grouped) {
        compact_streams_kernel<true><<<dim3((unsigned)cblocks), dim3(256), 0, s>>>(
            w.scratch, kStreamCap, o.offsets, o.lengths, nullptr, w.nstreams, o.payload, o.payload_cap, skew, o.status,
            w.group_sums, w.tile_sums);
    } else if (fused_scan) {
        if (int rc = launch_scan(w.tile_sums, cblocks, INT_MAX, w.tile_base, w.tile_scan_scratch, s)) return rc;
        compact_streams_kernel<true><<<dim3((unsigned)cblocks), dim3(256), 0, s>>>(
            w.scratch, kStreamCap, o.offsets, o.lengths, w.tile_base, w.nstreams, o.payload, o.payload_cap, skew, o.status);
    } else {
        if (int rc = launch_scan(o.lengths, w.nstreams, kStreamCap, o.offsets, w.scan_scratch, s)) return rc;
        compact_streams_kernel<false><<<dim3((unsigned)cblocks), dim3(256), 0, s>>>(
            w.scratch, kStreamCap, o.offsets, nullptr, nullptr, w.nstreams, o.payload, o.payload_cap, skew, o.status);
    }
    return check_launch("compact");
}

int check_kv_geometry(const char *what, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t chunk_tokens)
{
    if (int rc = check_dt(kv_dt, what)) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0) return fail(CG_ERR_ARG, "%s: empty input", what);
    if (chunk_tokens <= 0) return fail(CG_ERR_ARG, "%s: chunk_tokens must be positive", what);
    if (chunk_tokens > 65535) return fail(CG_ERR_ARG, "%s: at most 65535 tokens per chunk (16-bit counters)", what);
    // refused here, before the first launch of the call has written anything
    return check_grid_limits(2 * L, cg_num_subchunks(T, chunk_tokens));
}

// cg_encode_kv.  `flags` (CG_TEST_*, 0 from cg_encode_kv) switch the internal choices that have
// two forms to the form the call would not take by itself; the results are the same.
int encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
              int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
              int max_bins, int64_t chunk_tokens, int delta_group, int16_t *cdf, void *maxima,
              int32_t *lengths, int64_t *offsets, uint8_t *payload, int64_t payload_cap,
              int32_t *status, void *workspace, size_t workspace_bytes, void *stream, int flags)
{
    const bool four_bit_words = !(flags & CG_TEST_BYTE_SYMBOLS);
    if (!kv || !key_bins || !value_bins || !cdf || !maxima || !lengths || !offsets || !payload || !status || !workspace)
        return fail(CG_ERR_ARG, "encode_kv: null pointer");
    if (int rc = check_kv_geometry("encode_kv", kv_dt, L, T, H, D, chunk_tokens)) return rc;
    if (int rc = check_lp(max_bins + 1, "encode_kv")) return rc;
    if (delta_group < 0 || delta_group > kSub) return fail(CG_ERR_ARG, "encode_kv: delta_group must be in [0, %d]", kSub);
    const int64_t C = H * D;
    const EncodeWorkspace w(workspace, L, T, C, chunk_tokens, 1);
    if (workspace_bytes < w.total) return fail(CG_ERR_WORKSPACE, "encode_kv: workspace too small");
    if (!aligned_to(workspace, 256)) return fail(CG_ERR_ARG, "encode_kv: workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);
    const LevelOut o = {key_bins, value_bins, max_bins, cdf, lengths, offsets, payload, payload_cap, status};

    const bool packed = kv_vectorizable(kv, D, C, sl, skv, st, sh) && C % 8 == 0;
    if (delta_group > 0 && !packed)
        return fail(CG_ERR_ARG, "encode_kv: delta groups need head sizes and strides that are multiples of 8 and a 16-byte aligned tensor");
    if (packed) {
        uint32_t *sym4 = reinterpret_cast<uint32_t *>(w.symbols);
        const bool nibbles = four_bit_words && delta_group == 0;
        // The quantizer counts the symbols as it makes them and writes the tables, where the
        // tables fit its LDS and there are chunks enough to fill the GPU; the coder then only codes.
        QuantTablesShape shape;
        const int64_t nchunks = cg_num_chunks(T, chunk_tokens);
        const int64_t reach = chunk_tokens < T ? chunk_tokens : T;       // tokens of the longest chunk
        // Few (row, chunk) pairs but long chunks (one table over a whole context): the chunks are
        // cut into parts of whole sub-chunks, a block each, whose counters are summed in memory
        // (in the stream slots of the workspace, which nothing uses before the coder runs).
        int64_t part_tokens = 0;
        if ((flags & CG_TEST_SPLIT_CHUNKS) && reach > kSub) part_tokens = kSub;
        else if (2 * L * nchunks < kQuantTablesPartBlocks && reach > kSub) {
            const int64_t want = ceil_div(kQuantTablesPartBlocks, 2 * L * nchunks);     // parts per chunk
            part_tokens = reach / want / kSub * kSub;
            if (part_tokens < kSub) part_tokens = kSub;
        }
        const int64_t nparts = part_tokens ? ceil_div(reach, part_tokens) : 1;
        const bool enough_blocks = (flags & CG_TEST_TABLES_IN_QUANTIZER) || 2 * L * nchunks * nparts >= kQuantTablesMinBlocks;
        // the table builder addresses a chunk's token rows with a 32-bit offset from the chunk's first
        const bool addressable = st >= 0 && sh >= 0 && ((H - 1) * sh + (D - 1) + (reach - 1) * st) * 2 + 16 <= 0xFFFFFFF0ll;
        if (delta_group == 0 && !(flags & CG_TEST_TABLES_IN_CODER) && enough_blocks && addressable &&
            quantize_tables_shape(C / 8, max_bins + 1, sh == D, shape)) {
            const size_t slots_bytes = (size_t)w.ntiles * kSlotTile * kStreamCap;
            if (nparts > 1 && (size_t)nchunks * 2 * L * shape.lds > slots_bytes) part_tokens = 0;       // one block per chunk after all
            if (int rc = launch_quantize_tables(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, sym4, maxima,
                                                reinterpret_cast<uint16_t *>(cdf), w.nsub, chunk_tokens, nibbles, status, shape, s,
                                                nparts > 1 ? part_tokens : 0, nparts > 1 && part_tokens ? w.scratch : nullptr, slots_bytes,
                                                w.group_sums)) return rc;
            return code_and_compact(o, sym4, nullptr, w, L, T, C, chunk_tokens, s, maxima, kv_dt, nibbles, true);
        }
        if (int rc = launch_quantize_pack(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, sym4,
                                          maxima, w.nsub, chunk_tokens, delta_group, s, status, 0, nullptr, nullptr, 0,
                                          nibbles, nullptr, max_bins + 1)) return rc;
        return code_and_compact(o, sym4, nullptr, w, L, T, C, chunk_tokens, s, maxima, kv_dt, nibbles);
    }
    clear_status_kernel<<<1, 1, 0, s>>>(status);
    if (int rc = launch_quantize(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, w.symbols, maxima, s)) return rc;
    return code_and_compact(o, nullptr, w.symbols, w, L, T, C, chunk_tokens, s);
}

}  // namespace

extern "C" {

int cg_encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                 int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
                 int max_bins, int64_t chunk_tokens, int delta_group, int16_t *cdf, void *maxima,
                 int32_t *lengths, int64_t *offsets, uint8_t *payload, int64_t payload_cap,
                 int32_t *status, void *workspace, size_t workspace_bytes, void *stream)
{
    return encode_kv(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, max_bins, chunk_tokens, delta_group,
                     cdf, maxima, lengths, offsets, payload, payload_cap, status, workspace, workspace_bytes, stream, 0);
}

int cg_test_encode_kv(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                      int64_t skv, int64_t st, int64_t sh, const float *key_bins, const float *value_bins,
                      int max_bins, int64_t chunk_tokens, int delta_group, int16_t *cdf, void *maxima,
                      int32_t *lengths, int64_t *offsets, uint8_t *payload, int64_t payload_cap,
                      int32_t *status, void *workspace, size_t workspace_bytes, void *stream, int flags)
{
    return encode_kv(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins, value_bins, max_bins, chunk_tokens, delta_group,
                     cdf, maxima, lengths, offsets, payload, payload_cap, status, workspace, workspace_bytes, stream, flags);
}

int cg_encode_kv_levels(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D, int64_t sl,
                        int64_t skv, int64_t st, int64_t sh, int nlevels, const float *const *key_bins,
                        const float *const *value_bins, const int *max_bins, int64_t chunk_tokens,
                        int16_t *const *cdf, void *maxima, int32_t *const *lengths, int64_t *const *offsets,
                        uint8_t *const *payload, const int64_t *payload_cap, int32_t *status,
                        void *workspace, size_t workspace_bytes, void *stream)
{
    if (!kv || !key_bins || !value_bins || !max_bins || !cdf || !maxima || !lengths || !offsets || !payload ||
        !payload_cap || !status || !workspace)
        return fail(CG_ERR_ARG, "encode_kv_levels: null pointer");
    if (nlevels < 1 || nlevels > CG_MAX_LEVELS)
        return fail(CG_ERR_ARG, "encode_kv_levels: between 1 and %d levels, got %d", CG_MAX_LEVELS, nlevels);
    if (int rc = check_kv_geometry("encode_kv_levels", kv_dt, L, T, H, D, chunk_tokens)) return rc;
    int lp_lv[CG_MAX_LEVELS];
    for (int v = 0; v < nlevels; ++v) {
        if (!key_bins[v] || !value_bins[v] || !cdf[v] || !lengths[v] || !offsets[v] || !payload[v])
            return fail(CG_ERR_ARG, "encode_kv_levels: null pointer for level %d", v);
        if (int rc = check_lp(max_bins[v] + 1, "encode_kv_levels")) return rc;
        lp_lv[v] = max_bins[v] + 1;
    }
    const int64_t C = H * D;
    const EncodeWorkspace w(workspace, L, T, C, chunk_tokens, nlevels);
    if (workspace_bytes < w.total) return fail(CG_ERR_WORKSPACE, "encode_kv_levels: workspace too small");
    if (!aligned_to(workspace, 256)) return fail(CG_ERR_ARG, "encode_kv_levels: workspace must be 256-byte aligned");
    hipStream_t s = static_cast<hipStream_t>(stream);

    const bool packed = kv_vectorizable(kv, D, C, sl, skv, st, sh) && C % 8 == 0;
    if (packed) {
        // one pass over the tensor: every row is loaded once, its maximum found once, and its
        // symbols written once per level
        uint32_t *sym4 = reinterpret_cast<uint32_t *>(w.symbols);
        if (int rc = launch_quantize_pack(kv, kv_dt, L, T, H, D, sl, skv, st, sh, nullptr, nullptr, sym4, maxima,
                                          w.nsub, chunk_tokens, 0, s, status, nlevels, key_bins, value_bins,
                                          (int64_t)(w.symbols_bytes / 4), true, lp_lv)) return rc;
    }
    for (int v = 0; v < nlevels; ++v) {
        const LevelOut o = {key_bins[v], value_bins[v], max_bins[v], cdf[v], lengths[v], offsets[v],
                            payload[v], payload_cap[v], status + v};
        uint8_t *symbols = w.symbols + (size_t)v * w.symbols_bytes;
        if (packed) {
            if (int rc = code_and_compact(o, reinterpret_cast<uint32_t *>(symbols), nullptr, w, L, T, C, chunk_tokens, s, maxima, kv_dt, true)) return rc;
        } else {
            // shapes the vector loads cannot take: one plain quantization pass per level
            clear_status_kernel<<<1, 1, 0, s>>>(status + v);
            if (int rc = launch_quantize(kv, kv_dt, L, T, H, D, sl, skv, st, sh, key_bins[v], value_bins[v], symbols, maxima, s)) return rc;
            if (int rc = code_and_compact(o, nullptr, symbols, w, L, T, C, chunk_tokens, s)) return rc;
        }
    }
    return CG_OK;
}

int cg_decode_kv(const int16_t *cdf, int max_bins, const void *maxima, int max_dt, const int64_t *offsets,
                 const uint8_t *payload, int64_t payload_bytes, const float *key_bins,
                 const float *value_bins, int64_t L, int64_t T, int64_t H, int64_t D,
                 int64_t chunk_tokens, int delta_group, void *out, int out_dt, int64_t ol, int64_t okv,
                 int64_t ot, int64_t oh, void *stream)
{
    if (!cdf || !maxima || !offsets || !key_bins || !value_bins || !out || !payload)
        return fail(CG_ERR_ARG, "decode_kv: null pointer");
    if (int rc = check_dt(max_dt, "decode_kv")) return rc;
    if (int rc = check_dt(out_dt, "decode_kv")) return rc;
    if (L <= 0 || T <= 0 || H <= 0 || D <= 0 || chunk_tokens <= 0) return fail(CG_ERR_ARG, "decode_kv: empty input");
    if (int rc = check_lp(max_bins + 1, "decode_kv")) return rc;
    if (delta_group < 0 || delta_group > kSub) return fail(CG_ERR_ARG, "decode_kv: delta_group must be in [0, %d]", kSub);
    const int64_t C = H * D, rows = 2 * L;
    if (D > INT_MAX) return fail(CG_ERR_ARG, "decode_kv: head size too large");
    // the kernel stores through a buffer descriptor per block: a channel's byte offset plus a
    // token row's byte offset inside one stream's token range must fit 32 bits
    if (ot < 0 || oh < 0 || ((H - 1) * oh + (D - 1) + (int64_t)(kSub - 1) * ot) * 2 + 2 > 0xFFFFFFFFll)
        return fail(CG_ERR_ARG, "decode_kv: negative output strides, or %d token rows of one layer's keys or values "
                                "span 4 GiB or more", kSub);
    const int64_t nsub = cg_num_subchunks(T, chunk_tokens);
    // two wavefronts per block: a block's slot is held until its slowest wavefront is through
    // its 256 symbols, and smaller blocks leave fewer finished wavefronts waiting for that
    // (one wavefront per block loses more to the per-block set-up than it gains)
    int block = pick_block(C, max_bins + 1);
    if (block > 128) block = 128;
    DecodeArgs a;
    memset(&a, 0, sizeof(a));
    a.cdf = reinterpret_cast<const uint16_t *>(cdf);
    a.lp = max_bins + 1;
    if (int rc = set_byte_window(a, payload, payload_bytes, "decode_kv")) return rc;
    a.offsets = offsets;
    a.out_kv = static_cast<uint16_t *>(out);
    a.ol = ol;
    a.okv = okv;
    a.ot = ot;
    a.oh = oh;
    a.L = L;
    a.D = (int32_t)D;
    a.maxima = static_cast<const uint16_t *>(maxima);
    a.max_dt = max_dt;
    a.delta_group = delta_group;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    int64_t nblocks;
    if (int rc = make_grid(rows, C, T, chunk_tokens, nsub, block, a.sg, nblocks)) return rc;
    const size_t shmem = decode_shmem(a.lp, block);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid = stream_grid(a.sg, nblocks);
    // the blocks that are resident together at the launch's end (32 wavefronts per compute unit
    // where registers and LDS allow it, which they do for tables of up to 33 entries)
    const int64_t resident = (int64_t)compute_units() * (2048 / block);
    a.last_round_first = (uint32_t)(nblocks > resident ? nblocks - resident : 0);
    if (out_dt == CG_DT_BF16) CG_DISPATCH_BS(block, (launch_decode_kv_log2<BS, OUT_BF16>(a, grid, shmem, s)));
    else CG_DISPATCH_BS(block, (launch_decode_kv_log2<BS, OUT_F16>(a, grid, shmem, s)));
    return check_launch("decode_kv");
}

int cg_tables_to_counts(const int16_t *cdf, int max_bins, int64_t ngroups, int64_t C, const int32_t *tokens,
                        uint8_t *counts, int32_t *nsym, int32_t *inexact, void *stream)
{
    if (!cdf || !tokens || !counts || !nsym || !inexact) return fail(CG_ERR_ARG, "tables_to_counts: null pointer");
    if (int rc = check_lp(max_bins + 1, "tables_to_counts")) return rc;
    if (ngroups <= 0 || C <= 0 || ngroups > 65535) return fail(CG_ERR_ARG, "tables_to_counts: bad group or channel count");
    hipStream_t s = static_cast<hipStream_t>(stream);
    clear_ints_kernel<<<dim3((unsigned)ceil_div(ngroups, kWireThreads)), dim3(kWireThreads), 0, s>>>(nsym, ngroups, inexact);
    const dim3 grid((unsigned)ceil_div(C, kWireThreads), (unsigned)ngroups);
    tables_to_counts_kernel<<<grid, dim3(kWireThreads), 0, s>>>(reinterpret_cast<const uint16_t *>(cdf), max_bins + 1, C,
                                                               tokens, counts, nsym, inexact);
    return check_launch("tables_to_counts");
}

int cg_pack_counts(const uint8_t *counts, int max_bins, int64_t ngroups, int64_t C, const int32_t *nsym,
                   const int64_t *starts, uint8_t *out, void *stream)
{
    if (!counts || !nsym || !starts || !out) return fail(CG_ERR_ARG, "pack_counts: null pointer");
    if (int rc = check_lp(max_bins + 1, "pack_counts")) return rc;
    if (ngroups <= 0 || C <= 0 || ngroups > 65535) return fail(CG_ERR_ARG, "pack_counts: bad group or channel count");
    const dim3 grid((unsigned)ceil_div(C, kWireThreads), (unsigned)ngroups);
    pack_counts_kernel<<<grid, dim3(kWireThreads), 0, static_cast<hipStream_t>(stream)>>>(counts, max_bins + 1, C, nsym,
                                                                                         starts, out);
    return check_launch("pack_counts");
}

int cg_counts_to_tables(const uint8_t *data, int64_t data_bytes, int max_bins, int64_t ngroups, int64_t C,
                        const int32_t *tokens, const uint8_t *nsym, const int64_t *starts, int16_t *cdf,
                        int32_t *invalid, void *stream)
{
    if (!data || !tokens || !nsym || !starts || !cdf || !invalid) return fail(CG_ERR_ARG, "counts_to_tables: null pointer");
    if (int rc = check_lp(max_bins + 1, "counts_to_tables")) return rc;
    if (ngroups <= 0 || C <= 0 || ngroups > 65535 || data_bytes < 0)
        return fail(CG_ERR_ARG, "counts_to_tables: bad group or channel count");
    hipStream_t s = static_cast<hipStream_t>(stream);
    clear_ints_kernel<<<dim3(1), dim3(kWireThreads), 0, s>>>(invalid, 1, nullptr);
    const dim3 grid((unsigned)ceil_div(C, kWireThreads), (unsigned)ngroups);
    counts_to_tables_kernel<<<grid, dim3(kWireThreads), 0, s>>>(data, data_bytes, max_bins + 1, C, tokens, nsym, starts,
                                                               reinterpret_cast<uint16_t *>(cdf), invalid);
    return check_launch("counts_to_tables");
}

}  // extern "C"
