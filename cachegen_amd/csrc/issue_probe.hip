// Calibration probe of the CacheGen KV codec library for MI355X (gfx950): how fast one SIMD
// issues vector instructions, and at which engine clock.  Not part of the codec: bench.py uses it
// to price the decoder's instruction count against what this GPU really issues, at the clock it
// really runs at, instead of against 4 cycles per instruction at the data-sheet clock.
//
// The two range coders are bound by the issue of vector instructions.  On this GPU a wave64
// instruction takes a SIMD 4 cycles, except that adds, subtracts, bitwise operations, right
// shifts, moves and float32 add/multiply take 2 when their operands are registers (no scalar
// register, SDWA or DPP operand).  The probe measures both classes, and a sequence with the
// decoder's own mix and order of instructions, with 8 wavefronts per SIMD and two independent
// dependency chains per wavefront, and reads the engine clock from inside the kernel (the shader
// clock counter against the constant 100 MHz counter).
#include <hip/hip_runtime.h>

#include <cstdint>

extern "C" {

// kind: 0 = cheap class (v_add_u32, v_xor_b32, v_lshrrev_b32, v_and_b32 in turn)
//       1 = full-rate class (v_mul_u32_u24, v_cndmask_b32, v_lshlrev_b32, v_add3_u32 in turn)
//       2 = one decoded symbol of decode_streams_kernel (rows of at most 16 levels): 27 instructions
//           of the full class and 11 of the cheap class in the order the compiler emits them
// iters: loop trips of 64 (kinds 0, 1) or 76 (kind 2: two symbols of 38) instructions per wavefront
// ns_per_instruction: time one SIMD takes per wave64 instruction, 8 wavefronts resident
// clock_mhz: engine clock while the probe ran
// Returns 0, or the hipError_t that stopped it.
int cg_probe_issue_rate(int kind, int iters, double *ns_per_instruction, double *clock_mhz);

// The engine clock averaged over about `microseconds` of wall time, sampled by ONE wavefront that
// idles between two readings: launched on `stream` next to other work (a side stream of the
// benchmark), it reports the clock the GPU ran at while that work was running.  The result is
// read with cg_probe_clock_result after the stream has been synchronized.
int cg_probe_clock_start(int microseconds, void *stream);
int cg_probe_clock_result(double *clock_mhz, double *window_us);

}  // extern "C"

namespace {

struct ClockSample {
    uint64_t cycles0, ticks0, cycles1, ticks1;      // shader clock counter, 100 MHz counter
};

__device__ __forceinline__ void read_clocks(uint64_t &cycles, uint64_t &ticks)
{
    cycles = clock64();
    ticks = wall_clock64();
}

template <int KIND>
__global__ __launch_bounds__(256) void issue_rate_kernel(uint32_t *sink, ClockSample *sample, int iters, uint32_t seed)
{
    uint32_t a = threadIdx.x + seed, b = (blockIdx.x * 3 + 1) & 15, c = seed ^ 0x1234567u, d = a * 7 + 1;
    uint64_t w = ((uint64_t)a << 32) | b, w2 = ((uint64_t)c << 32) | d;
    uint64_t cycles0 = 0, ticks0 = 0;
    if (blockIdx.x == 0 && threadIdx.x == 0) read_clocks(cycles0, ticks0);
    for (int i = 0; i < iters; ++i) {
        if (KIND == 0) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                asm volatile("v_add_u32 %0, %0, %2\n\tv_add_u32 %1, %1, %2\n\t"
                             "v_xor_b32 %0, %0, %3\n\tv_xor_b32 %1, %1, %3\n\t"
                             "v_lshrrev_b32 %0, 1, %0\n\tv_lshrrev_b32 %1, 1, %1\n\t"
                             "v_and_b32 %0, %0, %3\n\tv_and_b32 %1, %1, %3"
                             : "+v"(a), "+v"(c) : "v"(b), "v"(d));
        } else if (KIND == 1) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
                asm volatile("v_mul_u32_u24 %0, %0, %2\n\tv_mul_u32_u24 %1, %1, %2\n\t"
                             "v_cndmask_b32 %0, %0, %3, vcc\n\tv_cndmask_b32 %1, %1, %3, vcc\n\t"
                             "v_lshlrev_b32 %0, 1, %0\n\tv_lshlrev_b32 %1, 1, %1\n\t"
                             "v_add3_u32 %0, %0, %2, %3\n\tv_add3_u32 %1, %1, %2, %3"
                             : "+v"(a), "+v"(c) : "v"(b), "v"(d) : "vcc");
        } else {
            // the symbol loop of decode_streams_kernel<128, 5, OFFSETS, F16>, rows of at most 16
            // levels, as compiled: search (two probes on registers, two on table entries), bounds
            // and the one test, dequantisation, state update, bit window; LDS reads and the store
            // left out (they are not vector-ALU instructions); twice, on two sets of registers
#define CG_PROBE_SYMBOL(x, y, p, q)                                                         \
            "v_mul_u32_u24 " p ", " x ", %8\n\tv_cmp_gt_u32 vcc, " p ", " y "\n\t"              \
            "v_cndmask_b32 " q ", %8, %9, vcc\n\tv_mul_u32_u24 " q ", " q ", " x "\n\t"         \
            "v_cndmask_b32 " p ", %9, 0, vcc\n\tv_cmp_gt_u32 vcc, " q ", " y "\n\t"             \
            "v_cndmask_b32 " q ", %8, 0, vcc\n\tv_add3_u32 " p ", %9, " p ", " q "\n\t"         \
            "v_add_u32 " q ", 0x208, " p "\n\tv_mul_u32_u24 " p ", " x ", " p "\n\t"            \
            "v_cmp_gt_u32 vcc, " p ", " y "\n\tv_cndmask_b32 " p ", " q ", " p ", vcc\n\t"      \
            "v_add_u32 " q ", 0x104, " p "\n\tv_mul_u32_u24 " p ", " x ", " p "\n\t"            \
            "v_cmp_gt_u32 vcc, " p ", " y "\n\tv_cndmask_b32 " p ", " q ", " p ", vcc\n\t"      \
            "v_add_u32 " q ", " p ", %9\n\t"                                                    \
            "v_mul_hi_u32 " p ", " p ", " x "\n\tv_mul_hi_u32 " q ", " q ", " x "\n\t"          \
            "v_sub_u32 " q ", " q ", " p "\n\tv_sub_u32 " y ", " y ", " p "\n\t"                \
            "v_cmp_ge_u32 vcc, " y ", " q "\n\t"                                                \
            "v_mul_f32 " p ", " p ", " q "\n\tv_cvt_f16_f32 " p ", " p "\n\t"                   \
            "v_add_u32 " p ", " p ", " x "\n\tv_add3_u32 " q ", " q ", " p ", -1\n\t"           \
            "v_xor_b32 " y ", " q ", " p "\n\tv_bitop3_b32 " q ", " q ", " p ", " q " bitop3:0xf3\n\t" \
            "v_ffbh_u32 " y ", " y "\n\tv_add_lshl_u32 " q ", " q ", " q ", " y "\n\t"          \
            "v_ffbh_u32 " q ", " q "\n\tv_add_u32 " q ", " q ", " y "\n\t"                      \
            "v_sub_co_u32 " p ", vcc, " p ", " q "\n\tv_lshlrev_b32 " x ", " q ", " x "\n\t"    \
            "v_mov_b32 " y ", " p "\n\tv_lshlrev_b32 " p ", " q ", " p "\n\t"
            uint32_t t0 = a, t1 = c, t2 = b, t3 = d;
            asm volatile(CG_PROBE_SYMBOL("%0", "%1", "%4", "%5")
                         "v_lshlrev_b64 %2, %5, %2\n\tv_lshlrev_b64 %3, %5, %3\n\t"
                         CG_PROBE_SYMBOL("%1", "%0", "%6", "%7")
                         "v_lshlrev_b64 %2, %7, %2\n\tv_lshlrev_b64 %3, %7, %3"
                         : "+v"(a), "+v"(c), "+v"(w), "+v"(w2), "+v"(t0), "+v"(t1), "+v"(t2), "+v"(t3)
                         : "v"(b), "v"(d)
                         : "vcc");
#undef CG_PROBE_SYMBOL
        }
    }
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        sample->cycles0 = cycles0;
        sample->ticks0 = ticks0;
        read_clocks(sample->cycles1, sample->ticks1);
    }
    sink[blockIdx.x * 256 + threadIdx.x] = a + c + d + (uint32_t)w + (uint32_t)(w >> 32) + (uint32_t)w2 + (uint32_t)(w2 >> 32);
}

// One wavefront that sleeps between two readings of the clocks, for about `ticks` ticks of the
// 100 MHz counter; bounded by that counter, so it always ends.
__global__ __launch_bounds__(64) void clock_window_kernel(ClockSample *sample, uint64_t ticks)
{
    uint64_t cycles0, ticks0, cycles1, ticks1;
    read_clocks(cycles0, ticks0);
    do {
        __builtin_amdgcn_s_sleep(64);
        read_clocks(cycles1, ticks1);
    } while (ticks1 - ticks0 < ticks);
    if (threadIdx.x == 0) {
        sample->cycles0 = cycles0;
        sample->ticks0 = ticks0;
        sample->cycles1 = cycles1;
        sample->ticks1 = ticks1;
    }
}

ClockSample *g_window = nullptr;        // the sampler's result, device memory kept for the process

}  // namespace

#define CG_PROBE_CHECK(x)                  \
    do {                                   \
        const hipError_t e_ = (x);         \
        if (e_ != hipSuccess) return (int)e_; \
    } while (0)

extern "C" int cg_probe_issue_rate(int kind, int iters, double *ns_per_instruction, double *clock_mhz)
{
    if (kind < 0 || kind > 2 || iters <= 0 || !ns_per_instruction || !clock_mhz) return (int)hipErrorInvalidValue;
    int dev = 0, cus = 0;
    CG_PROBE_CHECK(hipGetDevice(&dev));
    CG_PROBE_CHECK(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev));
    const int blocks = cus * 8 * 4;          // 8 blocks of 4 wavefronts per compute unit, 4 rounds
    uint32_t *sink = nullptr;
    ClockSample *sample = nullptr;
    CG_PROBE_CHECK(hipMalloc(&sink, (size_t)blocks * 256 * sizeof(uint32_t)));
    CG_PROBE_CHECK(hipMalloc(&sample, sizeof(ClockSample)));
    hipEvent_t e0, e1;
    CG_PROBE_CHECK(hipEventCreate(&e0));
    CG_PROBE_CHECK(hipEventCreate(&e1));
    float ms = 0.0f;
    for (int rep = 0; rep < 2; ++rep) {      // the first run brings the clock up
        CG_PROBE_CHECK(hipEventRecord(e0, nullptr));
        if (kind == 0) issue_rate_kernel<0><<<blocks, 256>>>(sink, sample, iters, rep + 1);
        else if (kind == 1) issue_rate_kernel<1><<<blocks, 256>>>(sink, sample, iters, rep + 1);
        else issue_rate_kernel<2><<<blocks, 256>>>(sink, sample, iters, rep + 1);
        CG_PROBE_CHECK(hipGetLastError());
        CG_PROBE_CHECK(hipEventRecord(e1, nullptr));
        CG_PROBE_CHECK(hipDeviceSynchronize());
        CG_PROBE_CHECK(hipEventElapsedTime(&ms, e0, e1));
    }
    ClockSample host;
    CG_PROBE_CHECK(hipMemcpy(&host, sample, sizeof(host), hipMemcpyDeviceToHost));
    CG_PROBE_CHECK(hipFree(sink));
    CG_PROBE_CHECK(hipFree(sample));
    CG_PROBE_CHECK(hipEventDestroy(e0));
    CG_PROBE_CHECK(hipEventDestroy(e1));
    const double per_trip = kind == 2 ? 76.0 : 64.0;     // instructions per loop trip and wavefront
    const double per_simd = (double)blocks * 4.0 * iters * per_trip / (cus * 4.0);
    *ns_per_instruction = (double)ms * 1e6 / per_simd;
    const double ticks = (double)(host.ticks1 - host.ticks0);
    *clock_mhz = ticks > 0 ? (double)(host.cycles1 - host.cycles0) / ticks * 100.0 : 0.0;
    return 0;
}

extern "C" int cg_probe_clock_start(int microseconds, void *stream)
{
    if (microseconds <= 0 || microseconds > 10 * 1000 * 1000) return (int)hipErrorInvalidValue;
    if (!g_window) CG_PROBE_CHECK(hipMalloc(&g_window, sizeof(ClockSample)));
    clock_window_kernel<<<1, 64, 0, static_cast<hipStream_t>(stream)>>>(g_window, (uint64_t)microseconds * 100u);
    return (int)hipGetLastError();
}

extern "C" int cg_probe_clock_result(double *clock_mhz, double *window_us)
{
    if (!g_window || !clock_mhz || !window_us) return (int)hipErrorInvalidValue;
    ClockSample host;
    CG_PROBE_CHECK(hipMemcpy(&host, g_window, sizeof(host), hipMemcpyDeviceToHost));
    const double ticks = (double)(host.ticks1 - host.ticks0);
    *window_us = ticks / 100.0;
    *clock_mhz = ticks > 0 ? (double)(host.cycles1 - host.cycles0) / ticks * 100.0 : 0.0;
    return 0;
}
