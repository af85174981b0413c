// Part of the CacheGen KV codec library for MI355X (gfx950); included by cachegen_hip.hip, which
// is the one translation unit.  Host-side launch helpers: block size, grids, kernel dispatch.
//
// Paths in the comments are relative to LMCache/ in the reference tree:
//   enc_new.cu = third_party/torchac_cuda/torchac_kernel_enc_new.cu
//   dec_new.cu = third_party/torchac_cuda/torchac_kernel_dec_new.cu
//   cal_cdf.cu = third_party/torchac_cuda/cal_cdf.cu
//   encoder.py = lmcache/storage_backend/serde/cachegen_encoder.py
//   decoder.py = lmcache/storage_backend/serde/cachegen_decoder.py
#pragma once

namespace {

// ------------------------------------------------------------------------------------
// host-side launch helpers
// ------------------------------------------------------------------------------------
// Lanes per block: as many adjacent channels as possible while the per-block table
// (lp words per lane) stays well inside the default dynamic LDS window.
int pick_block(int64_t nc, int lp)
{
    int block = 256;
    if (lp > 80) block = 128;
    while (block > 64 && nc <= block / 2) block /= 2;
    return block;
}

// The stream kernels run on a three-dimensional grid (channel tile, row, sub-chunk), so that a
// block reads its place from its index instead of dividing for it: rows and sub-chunks are grid
// dimensions and must fit one.
int check_grid_limits(int64_t rows, int64_t nsub)
{
    if (rows > 65535 || nsub > 65535)
        return fail(CG_ERR_ARG, "%lld rows and %lld sub-chunks: at most 65535 of each in one call", (long long)rows, (long long)nsub);
    return CG_OK;
}

int make_grid(int64_t rows, int64_t nc, int64_t T, int64_t S, int64_t nsub, int block,
              StreamGrid &sg, int64_t &nblocks)
{
    sg.rows = rows;
    sg.nc = nc;
    sg.ctiles = (int32_t)ceil_div(nc, block);
    sg.g.T = T;
    sg.g.S = S;
    sg.g.nsc = (int32_t)ceil_div(S, kSub);
    nblocks = nsub * rows * sg.ctiles;
    if (nblocks <= 0 || nblocks > INT_MAX) return fail(CG_ERR_ARG, "grid of %lld blocks is out of range", (long long)nblocks);
    return check_grid_limits(rows, nsub);
}

dim3 stream_grid(const StreamGrid &sg, int64_t nblocks)
{
    return dim3((unsigned)sg.ctiles, (unsigned)sg.rows, (unsigned)(nblocks / (sg.rows * sg.ctiles)));
}

// Run `launch` with the block size as a compile-time constant.
#define CG_DISPATCH_BS(block, ...)                      \
    do {                                                \
        if ((block) == 256) { constexpr int BS = 256; __VA_ARGS__; } \
        else if ((block) == 128) { constexpr int BS = 128; __VA_ARGS__; } \
        else { constexpr int BS = 64; __VA_ARGS__; }    \
    } while (0)

// key_bins, value_bins (packed symbols only, may be null): the rows of at most 15 symbols hold
// four bits a symbol.
int launch_cdf(const uint8_t *sym, const uint32_t *sym4, int64_t nsub, int64_t rows, int64_t T,
               int64_t nc, int64_t s0, int64_t s1, int64_t s2, int max_bins, int64_t S,
               uint16_t *cdf, hipStream_t stream, const float *key_bins = nullptr, const float *value_bins = nullptr)
{
    int block = pick_block(nc, max_bins + 1);
    while (!sym4 && block > 64 && (size_t)(max_bins + 1) * (block + 1) * sizeof(uint32_t) > 64 * 1024) block /= 2;
    CdfArgs a;
    a.sym = sym;
    a.s0 = s0;
    a.s1 = s1;
    a.s2 = s2;
    a.sym4 = sym4;
    a.nsub = nsub;
    a.nibbles = (sym4 && key_bins && value_bins) ? 1 : 0;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    a.L = rows / 2;
    a.cdf = cdf;
    a.rows = rows;
    a.nc = nc;
    a.ctiles = (int32_t)ceil_div(nc, block);
    a.max_bins = max_bins;
    a.g.T = T;
    a.g.S = S;
    a.g.nsc = (int32_t)ceil_div(S, kSub);
    const int64_t nblocks = ceil_div(T, S) * rows * a.ctiles;
    if (nblocks <= 0 || nblocks > INT_MAX) return fail(CG_ERR_ARG, "calculate_cdf: grid out of range");
    const size_t shmem = sym4 ? (size_t)(max_bins + 1) * (block + 2) * sizeof(uint16_t)
                              : (size_t)(max_bins + 1) * (block + 1) * sizeof(uint32_t);     // TableStride
    const dim3 grid((unsigned)nblocks), blk(block);
    if (sym4) CG_DISPATCH_BS(block, (calculate_cdf_kernel<BS, true><<<grid, blk, shmem, stream>>>(a)));
    else CG_DISPATCH_BS(block, (calculate_cdf_kernel<BS, false><<<grid, blk, shmem, stream>>>(a)));
    return check_launch("calculate_cdf");
}

int launch_scan(const int32_t *lengths, int64_t n, int32_t clamp, int64_t *offsets, void *scratch,
                hipStream_t stream)
{
    const int64_t ntiles = ceil_div(n, kScanTile);
    int64_t *sums = static_cast<int64_t *>(scratch);
    if (ntiles > 1 && n <= kScanSmallMax) {
        // a few thousand values: one block does it all, two launches fewer
        scan_small_kernel<<<dim3(1), dim3(kScanSmallThreads), 0, stream>>>(lengths, (int32_t)n, clamp, offsets);
        return check_launch("scan_lengths");
    }
    if (ntiles == 1) {
        scan_apply_kernel<<<dim3(1), dim3(kScanThreads), 0, stream>>>(lengths, n, clamp, nullptr, offsets);
        return check_launch("scan_lengths");
    }
    scan_tile_sums_kernel<<<dim3((unsigned)ntiles), dim3(kScanThreads), 0, stream>>>(lengths, n, clamp, sums);
    scan_sums_kernel<<<dim3(1), dim3(kScanThreads), 0, stream>>>(sums, ntiles);
    scan_apply_kernel<<<dim3((unsigned)ntiles), dim3(kScanThreads), 0, stream>>>(lengths, n, clamp, sums, offsets);
    return check_launch("scan_lengths");
}

int check_dt(int dt, const char *what)
{
    if (dt != CG_DT_F16 && dt != CG_DT_BF16) return fail(CG_ERR_ARG, "%s: dtype must be CG_DT_F16 or CG_DT_BF16", what);
    return CG_OK;
}

int check_lp(int lp, const char *what)
{
    if (lp < 2 || lp > CG_MAX_LP) return fail(CG_ERR_ARG, "%s: CDF length should be in [2, %d], got %d", what, CG_MAX_LP, lp);
    return CG_OK;
}

bool kv_vectorizable(const void *kv, int64_t D, int64_t C, int64_t sl, int64_t skv, int64_t st, int64_t sh)
{
    return (D % 8 == 0) && (sl % 8 == 0) && (skv % 8 == 0) && (st % 8 == 0) && (sh % 8 == 0) &&
           aligned_to(kv, 16) && (C / 8 <= 64 * kMaxUnits);
}

int launch_quantize(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                    int64_t sl, int64_t skv, int64_t st, int64_t sh, const float *key_bins,
                    const float *value_bins, uint8_t *sym, void *maxima, hipStream_t stream)
{
    const int64_t C = H * D;
    const int64_t nrows = 2 * L * T;
    const int64_t nblocks = ceil_div(nrows, 4);
    if (nblocks > INT_MAX || C > INT_MAX) return fail(CG_ERR_ARG, "quantize: tensor too large for one launch");
    const bool vec = kv_vectorizable(kv, D, C, sl, skv, st, sh) && aligned_to(sym, 8);
    const uint16_t *p = static_cast<const uint16_t *>(kv);
    uint16_t *mx = static_cast<uint16_t *>(maxima);
    dim3 grid((unsigned)nblocks), block(256);
    if (vec) {
        const int nunits = (int)(C / 8);
        const bool contiguous = (sh == D);
#define CG_LAUNCH_Q(DT, HC) quantize_kv_kernel<DT, HC><<<grid, block, 0, stream>>>( \
        p, L, T, (int)D, sl, skv, st, sh, key_bins, value_bins, sym, mx, nunits, nrows)
        if (kv_dt == CG_DT_F16) { if (contiguous) CG_LAUNCH_Q(CG_DT_F16, true); else CG_LAUNCH_Q(CG_DT_F16, false); }
        else { if (contiguous) CG_LAUNCH_Q(CG_DT_BF16, true); else CG_LAUNCH_Q(CG_DT_BF16, false); }
#undef CG_LAUNCH_Q
    } else {
        if (kv_dt == CG_DT_F16)
            quantize_kv_generic_kernel<CG_DT_F16><<<grid, block, 0, stream>>>(
                p, L, T, (int)D, (int)C, sl, skv, st, sh, key_bins, value_bins, sym, mx, nrows);
        else
            quantize_kv_generic_kernel<CG_DT_BF16><<<grid, block, 0, stream>>>(
                p, L, T, (int)D, (int)C, sl, skv, st, sh, key_bins, value_bins, sym, mx, nrows);
    }
    return check_launch("quantize_kv");
}

template <int DT, bool HC>
void launch_quantize_pack_nu(const PackedQuantArgs &a, int64_t nblocks, hipStream_t stream)
{
    const dim3 grid((unsigned)nblocks), block(256);
    if (a.delta_group > 0) {
        if (a.nunits <= 128) quantize_pack_delta_kernel<DT, HC, 2><<<grid, block, 0, stream>>>(a);
        else if (a.nunits <= 256) quantize_pack_delta_kernel<DT, HC, 4><<<grid, block, 0, stream>>>(a);
        else quantize_pack_delta_kernel<DT, HC, 8><<<grid, block, 0, stream>>>(a);
        return;
    }
    if (a.nlevels > 0) {
        if (a.nunits <= 128) quantize_pack_kernel<DT, HC, 2, true><<<grid, block, 0, stream>>>(a);
        else if (a.nunits <= 256) quantize_pack_kernel<DT, HC, 4, true><<<grid, block, 0, stream>>>(a);
        else quantize_pack_kernel<DT, HC, 8, true><<<grid, block, 0, stream>>>(a);
        return;
    }
    if (a.nunits <= 128) quantize_pack_kernel<DT, HC, 2><<<grid, block, 0, stream>>>(a);
    else if (a.nunits <= 256) quantize_pack_kernel<DT, HC, 4><<<grid, block, 0, stream>>>(a);
    else quantize_pack_kernel<DT, HC, 8><<<grid, block, 0, stream>>>(a);
}

// nlevels > 0: key_bins_lv / value_bins_lv hold that many bins vectors and level v's words go
// to sym4 + v * level_words (one read of the tensor for all levels); nlevels == 0: one level,
// key_bins / value_bins.
int launch_quantize_pack(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                         int64_t sl, int64_t skv, int64_t st, int64_t sh, const float *key_bins,
                         const float *value_bins, uint32_t *sym4, void *maxima, int64_t nsub,
                         int64_t S, int delta_group, hipStream_t stream, int32_t *status, int nlevels = 0,
                         const float *const *key_bins_lv = nullptr, const float *const *value_bins_lv = nullptr,
                         int64_t level_words = 0, bool nibbles = false, const int *lp_lv = nullptr, int lp = 0)
{
    PackedQuantArgs a;
    memset(&a, 0, sizeof(a));
    // status: one word per level (one word when nlevels == 0), consecutive
    a.nstatus = nlevels > 0 ? nlevels : 1;
    for (int v = 0; v < a.nstatus; ++v) a.status[v] = status + v;
    a.nlevels = nlevels;
    for (int v = 0; v < nlevels; ++v) {
        a.key_bins_lv[v] = key_bins_lv[v];
        a.value_bins_lv[v] = value_bins_lv[v];
        a.lp_lv[v] = lp_lv ? lp_lv[v] : 0;
    }
    a.lp = lp;
    a.level_words = level_words;
    a.nibbles = nibbles ? 1 : 0;
    a.kv = static_cast<const uint16_t *>(kv);
    a.L = L;
    a.sl = sl;
    a.skv = skv;
    a.st = st;
    a.sh = sh;
    a.D = (int32_t)D;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    a.sym4 = sym4;
    a.maxima = static_cast<uint16_t *>(maxima);
    a.nunits = (int32_t)(H * D / 8);
    a.nsub = nsub;
    a.delta_group = delta_group;
    a.g.T = T;
    a.g.S = S;
    a.g.nsc = (int32_t)ceil_div(S, kSub);
    const int64_t nblocks = 2 * L * nsub * 16;
    if (nblocks > INT_MAX) return fail(CG_ERR_ARG, "quantize: tensor too large for one launch");
    const bool contiguous = (sh == D);
    if (kv_dt == CG_DT_F16) {
        if (contiguous) launch_quantize_pack_nu<CG_DT_F16, true>(a, nblocks, stream);
        else launch_quantize_pack_nu<CG_DT_F16, false>(a, nblocks, stream);
    } else {
        if (contiguous) launch_quantize_pack_nu<CG_DT_BF16, true>(a, nblocks, stream);
        else launch_quantize_pack_nu<CG_DT_BF16, false>(a, nblocks, stream);
    }
    return check_launch("quantize_pack");
}

// The quantizer that also builds the tables (quantize_tables_kernel): which of its forms takes a tensor of `nunits` units of 8 channels and tables of `lp` entries,
// if any.
// Long chunks of a call with fewer (row, chunk) pairs than this are cut into parts, whole
// sub-chunks each, until the launch has about this many blocks (measured on one table over
// 8192 tokens of 32 layers: parts of 256 tokens 0.765 ms, of 512 tokens 0.807, the whole encode).
constexpr int64_t kQuantTablesPartBlocks = 2048;

struct QuantTablesShape {
    int nu, lp;
    size_t lds;
};

constexpr size_t kMaxLdsPerBlock = 160 * 1024;      // gfx950
// fewer (row, chunk) blocks than this leave compute units idle: the two-kernel form is used instead
constexpr int64_t kQuantTablesMinBlocks = 512;

bool quantize_tables_shape(int64_t nunits, int lp, bool heads_contiguous, QuantTablesShape &shape)
{
    // 2048 channels: only tensors whose heads follow one another (the other form runs out of registers)
    const int nu = nunits <= 64 ? 1 : nunits <= 128 ? 2 : (nunits <= 256 && heads_contiguous) ? 4 : 0;
    if (!nu || (lp != 9 && lp != 17 && lp != 33 && lp != 65)) return false;
    shape.nu = nu;
    shape.lp = lp;
    shape.lds = (size_t)nu * 4 * lp * 256;
    return shape.lds <= kMaxLdsPerBlock;
}

// A kernel that wants more than 64 KiB of dynamic LDS has to be allowed to, once per device;
// `asked` holds one bit per device for that kernel.
int allow_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &asked)
{
    if (bytes <= 64 * 1024) return CG_OK;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return fail(CG_ERR_LAUNCH, "quantize_tables: hipGetDevice");
    if (asked.load(std::memory_order_relaxed) >> dev & 1) return CG_OK;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e != hipSuccess) return fail(CG_ERR_LAUNCH, "quantize_tables: hipFuncSetAttribute: %s", hipGetErrorString(e));
    asked.fetch_or(1ull << dev, std::memory_order_relaxed);
    return CG_OK;
}

template <int DT, bool HC, int NU, int LP>
int launch_quantize_tables_form(const QuantTablesArgs &a, dim3 grid, hipStream_t stream)
{
    typedef CountLayout<NU, LP> Layout;
    if (Layout::kBytes > (int)kMaxLdsPerBlock) return fail(CG_ERR_ARG, "quantize_tables: tables do not fit the LDS");
    static std::atomic<uint64_t> asked{0}, asked_for_sums{0};       // per form of the kernel: these are templates
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(&quantize_tables_kernel<DT, HC, NU, LP>), Layout::kBytes, asked)) return rc;
    if (!a.partial) {
        quantize_tables_kernel<DT, HC, NU, LP><<<grid, dim3(QuantTablesBlock<NU>::kThreads), Layout::kBytes, stream>>>(a);
        return check_launch("quantize_tables");
    }
    // chunks cut into parts: counters summed in memory, then one block per (chunk, row) for the tables
    if (int rc = allow_dynamic_lds(reinterpret_cast<const void *>(&tables_from_partial_kernel<NU, LP>), Layout::kBytes, asked_for_sums)) return rc;
    const int64_t nquads = (int64_t)grid.x * grid.y * (Layout::kBytes / 16);
    clear_quads_kernel<<<dim3((unsigned)ceil_div(nquads, 256)), dim3(256), 0, stream>>>(reinterpret_cast<uint4 *>(a.partial), nquads);
    quantize_tables_kernel<DT, HC, NU, LP><<<grid, dim3(QuantTablesBlock<NU>::kThreads), Layout::kBytes, stream>>>(a);
    tables_from_partial_kernel<NU, LP><<<dim3(grid.x, grid.y), dim3(QuantTablesBlock<NU>::kThreads), Layout::kBytes, stream>>>(
        a.partial, a.cdf, a.nunits, a.g);
    return check_launch("quantize_tables");
}

template <int DT, bool HC, int LP>
int launch_quantize_tables_nu(const QuantTablesArgs &a, const QuantTablesShape &shape, dim3 grid, hipStream_t stream)
{
    if (shape.nu == 1) return launch_quantize_tables_form<DT, HC, 1, LP>(a, grid, stream);
    if (shape.nu == 2) return launch_quantize_tables_form<DT, HC, 2, LP>(a, grid, stream);
    if (HC && LP <= 33) return launch_quantize_tables_form<DT, true, 4, (LP <= 33 ? LP : 33)>(a, grid, stream);
    return fail(CG_ERR_ARG, "quantize_tables: shape not built");
}

template <int DT, bool HC>
int launch_quantize_tables_shape(const QuantTablesArgs &a, const QuantTablesShape &shape, dim3 grid, hipStream_t stream)
{
    switch (shape.lp) {
    case 9: return launch_quantize_tables_nu<DT, HC, 9>(a, shape, grid, stream);
    case 17: return launch_quantize_tables_nu<DT, HC, 17>(a, shape, grid, stream);
    case 33: return launch_quantize_tables_nu<DT, HC, 33>(a, shape, grid, stream);
    case 65: return launch_quantize_tables_nu<DT, HC, 65>(a, shape, grid, stream);
    }
    return fail(CG_ERR_ARG, "quantize_tables: shape not built");
}

// Quantization, row maxima, packed symbols and the tables of every chunk in one launch.
int launch_quantize_tables(const void *kv, int kv_dt, int64_t L, int64_t T, int64_t H, int64_t D,
                           int64_t sl, int64_t skv, int64_t st, int64_t sh, const float *key_bins,
                           const float *value_bins, uint32_t *sym4, void *maxima, uint16_t *cdf, int64_t nsub, int64_t S,
                           bool nibbles, int32_t *status,
                           const QuantTablesShape &shape, hipStream_t stream,
                           int64_t part_tokens = 0, void *partial = nullptr, size_t partial_bytes = 0,
                           int32_t *group_sums = nullptr)
{
    QuantTablesArgs a;
    memset(&a, 0, sizeof(a));
    a.kv = static_cast<const uint16_t *>(kv);
    a.L = L;
    a.sl = sl;
    a.skv = skv;
    a.st = st;
    a.sh = sh;
    a.D = (int32_t)D;
    a.key_bins = key_bins;
    a.value_bins = value_bins;
    a.status = status;
    a.group_sums = group_sums;          // kMaxTileGroups words of the workspace
    a.ngroups = kMaxTileGroups;
    a.sym4 = sym4;
    a.maxima = static_cast<uint16_t *>(maxima);
    a.cdf = cdf;
    a.nunits = (int32_t)(H * D / 8);
    a.nsub = nsub;
    a.nibbles = nibbles ? 1 : 0;
    a.g.T = T;
    a.g.S = S;
    a.g.nsc = (int32_t)ceil_div(S, kSub);
    const int64_t nchunks = ceil_div(T, S);
    if (nchunks > INT_MAX || 2 * L > 65535) return fail(CG_ERR_ARG, "quantize_tables: grid out of range");
    dim3 grid((unsigned)nchunks, (unsigned)(2 * L));
    if (partial) {
        const int64_t nparts = ceil_div(S < T ? S : T, part_tokens);
        if (part_tokens <= 0 || part_tokens % kSub || nparts > 65535 || !aligned_to(partial, 16) ||
            (size_t)nchunks * 2 * L * shape.lds > partial_bytes)
            return fail(CG_ERR_ARG, "quantize_tables: parts of chunks out of range");
        grid.z = (unsigned)nparts;
        a.part_tokens = (int32_t)part_tokens;
        a.partial = static_cast<uint32_t *>(partial);
    }
    const bool contiguous = (sh == D);
    if (kv_dt == CG_DT_F16) {
        if (contiguous) return launch_quantize_tables_shape<CG_DT_F16, true>(a, shape, grid, stream);
        return launch_quantize_tables_shape<CG_DT_F16, false>(a, shape, grid, stream);
    }
    if (contiguous) return launch_quantize_tables_shape<CG_DT_BF16, true>(a, shape, grid, stream);
    return launch_quantize_tables_shape<CG_DT_BF16, false>(a, shape, grid, stream);
}

// Compute units of the current device (asked once per device).
int compute_units()
{
    static std::atomic<int> known[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = known[dev].load(std::memory_order_relaxed);
    if (!n) {
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        known[dev].store(n, std::memory_order_relaxed);
    }
    return n;
}

// Describe the readable byte window [bytes, bytes + nbytes) to the bit reader, which
// loads aligned words at 32-bit offsets from the window's 4-byte-aligned base.
int set_byte_window(DecodeArgs &a, const uint8_t *bytes, int64_t nbytes, const char *what)
{
    if (nbytes <= 0) return fail(CG_ERR_ARG, "%s: empty byte buffer", what);
    const uint32_t skew = (uint32_t)(reinterpret_cast<uintptr_t>(bytes) & 3u);
    a.bytes = bytes - skew;
    a.bytes_skew = skew;
    a.last_word = (skew + nbytes - 1) & ~3ll;
    return CG_OK;
}

size_t decode_shmem(int lp, int block) { return align_up((size_t)lp * block * sizeof(uint16_t), 4) + (size_t)(lp + kSub) * sizeof(float); }

// Tables of 2^k symbols (lp = 2^k + 1) take the kernel with the unrolled search.
template <int BS, int SRC, int OUT>
void launch_decode_log2(const DecodeArgs &a, dim3 grid, size_t shmem, hipStream_t stream)
{
    const dim3 blk(BS);
    switch (a.lp) {
    case 9: decode_streams_kernel<BS, 3, SRC, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 17: decode_streams_kernel<BS, 4, SRC, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 33: decode_streams_kernel<BS, 5, SRC, OUT><<<grid, blk, shmem, stream>>>(a); break;
    case 65: decode_streams_kernel<BS, 6, SRC, OUT><<<grid, blk, shmem, stream>>>(a); break;
    default: decode_streams_kernel<BS, -1, SRC, OUT><<<grid, blk, shmem, stream>>>(a); break;
    }
}

template <int SRC>
int launch_decode_symbols(const DecodeArgs &a, int64_t nblocks, int block, hipStream_t stream)
{
    const dim3 grid = stream_grid(a.sg, nblocks);
    const size_t shmem = decode_shmem(a.lp, block);
    CG_DISPATCH_BS(block, (launch_decode_log2<BS, SRC, OUT_SYMBOLS>(a, grid, shmem, stream)));
    return check_launch("decode");
}

template <int BS, int OUT>
void launch_decode_kv_log2(const DecodeArgs &a, dim3 grid, size_t shmem, hipStream_t stream)
{
    launch_decode_log2<BS, SRC_OFFSETS, OUT>(a, grid, shmem, stream);
}

}  // namespace
