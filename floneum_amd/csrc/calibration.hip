// Calibration kernels for the benchmark: what the matrix cores deliver with nothing else in the way.
//
// mfma_burn_kernel: one wavefront per SIMD of every compute unit runs rounds of 32 independent-accumulator
// v_mfma_f32_32x32x16 instructions on operands held in registers (no LDS, no memory traffic, no vector work), the
// instruction and the per-tile count of the prefill kernel's matrix phase.  Between rounds the wavefront may sleep so
// that the matrix pipe is busy only a given share of the time.  Operands are pseudo-random f16/bf16 values in
// (-2, 2), or all zero.  Every workgroup reports its shader-clock cycles and the 100 MHz wall-clock ticks it ran:
// the ratio is the clock the chip held under that load.  The figure bounds from above what ANY f16 kernel can reach
// on the same data; it has no counterpart in the reference.
#include "common.h"
#include "device_utils.h"

namespace fhip {

template <typename T>
struct BurnMma;
template <>
struct BurnMma<half_t> {
    typedef half8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ half_t from(float x) { return (half_t)x; }
};
template <>
struct BurnMma<bf16_t> {
    typedef bf16x8_t vec8;
    static __device__ __forceinline__ float16_t mfma(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static __device__ __forceinline__ __bf16 from(float x) { return (__bf16)x; }
};

// SLEEP: s_sleep units (64 cycles each) after every round of 32 MFMAs (1024 matrix-pipe cycles)
template <typename T, int SLEEP>
__global__ __launch_bounds__(256) void mfma_burn_kernel(float *sink, uint64_t *ticks, int rounds, int random_operands) {
    typedef typename BurnMma<T>::vec8 vec8;
    const uint64_t c0 = clock64(), w0 = wall_clock64();
    vec8 av[8], bv[4];
    uint32_t s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            s = s * 1664525u + 1013904223u;
            const float x = ((s >> 8) & 0xffff) / 65536.0f - 0.5f;
            s = s * 1664525u + 1013904223u;
            const float y = ((s >> 8) & 0xffff) / 65536.0f - 0.5f;
            av[j][i] = BurnMma<T>::from(random_operands ? x * 4.0f : 0.0f);
            bv[j & 3][i] = BurnMma<T>::from(random_operands ? y * 4.0f : 0.0f);
        }
    float16_t acc[4];
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[c][r] = 0.0f;
    for (int it = 0; it < rounds; it++) {
#pragma unroll
        for (int u = 0; u < 8; u++)
#pragma unroll
            for (int c = 0; c < 4; c++) acc[c] = BurnMma<T>::mfma(av[u], bv[c], acc[c]);
        if constexpr (SLEEP > 0) __builtin_amdgcn_s_sleep(SLEEP);
    }
    float res = 0.0f;
#pragma unroll
    for (int c = 0; c < 4; c++)
#pragma unroll
        for (int r = 0; r < 16; r++) res += acc[c][r];
    const uint64_t c1 = clock64(), w1 = wall_clock64();
    sink[blockIdx.x * 256 + threadIdx.x] = res;
    if (threadIdx.x == 0) {
        ticks[2 * blockIdx.x] = c1 - c0;
        ticks[2 * blockIdx.x + 1] = w1 - w0;
    }
}

// s_sleep units per round that leave the matrix pipe busy about `duty` percent of the time
static int sleep_units(int duty) {
    if (duty >= 100) return 0;
    const int idle_cycles = 1024 * (100 - duty) / duty;
    int units = (idle_cycles + 32) / 64;
    return units < 1 ? 1 : units > 15 ? 15 : units;
}

template <typename T>
static int launch_burn_t(int units, dim3 grid, hipStream_t stream, float *sink, uint64_t *ticks, int rounds, int random_operands) {
#define FHIP_BURN(U) \
    case U: hipLaunchKernelGGL((mfma_burn_kernel<T, U>), grid, dim3(256), 0, stream, sink, ticks, rounds, random_operands); break
    switch (units) {
        FHIP_BURN(0); FHIP_BURN(1); FHIP_BURN(2); FHIP_BURN(3); FHIP_BURN(4); FHIP_BURN(5); FHIP_BURN(6); FHIP_BURN(7);
        FHIP_BURN(8); FHIP_BURN(9); FHIP_BURN(10); FHIP_BURN(11); FHIP_BURN(12); FHIP_BURN(13); FHIP_BURN(14); FHIP_BURN(15);
        default: set_error("calibration: bad sleep count %d", units); return FHIP_ERR_INVALID_ARG;
    }
#undef FHIP_BURN
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

// read_burn_kernel: nothing but the loads of a streaming kernel.  Every workgroup reads its contiguous share of the
// buffer with 16-byte non-temporal loads, eight in flight per lane (a wavefront load instruction covers 1 KB, as in the
// decode kernels), folds what it read into one word and writes that word only if it has a value no fold produces.
__global__ __launch_bounds__(256) void read_burn_kernel(const uint4_t *src, size_t n16, uint32_t *sink) {
    const size_t per_wg = (n16 + gridDim.x - 1) / gridDim.x;
    const size_t lo = (size_t)blockIdx.x * per_wg, hi = lo + per_wg < n16 ? lo + per_wg : n16;
    uint32_t acc = 0;
    constexpr int U = 8;
    for (size_t base = lo + threadIdx.x; base < hi; base += (size_t)U * 256) {
        uint4_t v[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            const size_t i = base + (size_t)u * 256;
            v[u] = __builtin_nontemporal_load(src + (i < hi ? i : hi - 1));
        }
#pragma unroll
        for (int u = 0; u < U; u++) acc ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
    if (acc == 0x9e3779b9u && lo == hi) sink[blockIdx.x] = acc;  // never true (lo < hi whenever something was read)
}

int launch_calibration_read(const void *src, size_t bytes, int compute_units, void *sink, hipStream_t stream) {
    const size_t n16 = bytes / 16;
    if (n16 == 0) return FHIP_OK;
    const unsigned wgs = (unsigned)compute_units * 8;  // two rounds of four resident workgroups per CU
    hipLaunchKernelGGL(read_burn_kernel, dim3(wgs), dim3(256), 0, stream, (const uint4_t *)src, n16, (uint32_t *)sink);
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

// issue_probe_kernel: what ONE wavefront per SIMD can issue beside its matrix instructions.  A wavefront issues in order,
// so in a kernel that runs a single wavefront per SIMD (attn_prefill_mfma_rows32.hip: Q and O^T of 32 rows at head_dim
// 256 leave no registers for a second one) everything that is not a matrix instruction either fits into the 32 cycles
// the matrix pipe is busy with the last one or is paid for in full.  The loop is steps of one v_mfma_f32_32x32x16_f16
// on independent accumulators plus the companions `MIX` names, fenced so that the compiler keeps the steps apart; values
// read from LDS are used eight steps later, as operands or by a vector instruction.
template <int MIX>
__global__ __launch_bounds__(256, 1) void issue_probe_kernel(float *sink, uint64_t *ticks, int rounds) {
    __shared__ __attribute__((aligned(16))) char smem[49152];
    auto lds = (__attribute__((address_space(3))) char *)smem;
    for (int i = threadIdx.x; i < 49152 / 4; i += 256) ((__attribute__((address_space(3))) float *)lds)[i] = 1.0f;
    __syncthreads();
    const uint64_t c0 = clock64(), w0 = wall_clock64();
    const int lane = threadIdx.x & 63;
    float16_t acc[8];
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) acc[i][r] = 0.0f;
    half8_t a, b;
#pragma unroll
    for (int e = 0; e < 8; e++) a[e] = (half_t)(0.25f + 0.125f * e), b[e] = (half_t)0.5f;
    float x[8];
#pragma unroll
    for (int i = 0; i < 8; i++) x[i] = 1.0f + i;
    int addr = lane * 16;
    asm volatile("" : "+v"(addr));  // one address register, immediate offsets
    uint4_t la[8], lb[8], lc[8];
    short4_t tr[8][2];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        la[i] = lb[i] = lc[i] = uint4_t{0, 0, 0, 0};
        tr[i][0] = tr[i][1] = short4_t{0, 0, 0, 0};
    }
    int sacc = rounds;
    constexpr bool OPERAND_FROM_LDS = MIX == 6 || MIX == 7 || MIX == 9 || MIX == 10 || MIX == 11 || MIX == 12;
    for (int it = 0; it < rounds; it++) {
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const int i = k & 7;
            if (MIX == 1) acc[0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[0], 0, 0, 0);  // a dependent chain
            else if (OPERAND_FROM_LDS) acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, la[i]), b, acc[i], 0, 0, 0);
            else acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[i], 0, 0, 0);
            if (MIX == 2 || MIX == 3) {
#pragma unroll
                for (int j = 0; j < (MIX == 2 ? 4 : 8); j++) x[j] = __builtin_fmaf(x[j], 1.0001f, 0.5f);
            }
            if (MIX == 4) {
#pragma unroll
                for (int j = 0; j < 4; j++) x[j] = __builtin_amdgcn_exp2f(x[j]);
            }
            if (MIX == 5) {
#pragma unroll
                for (int j = 0; j < 4; j++) asm volatile("s_add_u32 %0, %0, 3" : "+s"(sacc) : : "scc");
            }
            if (OPERAND_FROM_LDS) la[i] = *(__attribute__((address_space(3))) uint4_t *)(lds + addr + i * 1024);
            if (MIX == 7) {
                lb[i] = *(__attribute__((address_space(3))) uint4_t *)(lds + 8192 + addr + i * 1024);
                lc[i] = *(__attribute__((address_space(3))) uint4_t *)(lds + 16384 + addr + i * 1024);
            }
            if (MIX == 8 || MIX == 9 || MIX == 10) {
                // (what the transposing reads of eight steps ago brought is consumed first)
                x[i] += __builtin_bit_cast(float, (int)tr[i][0][0] | ((int)tr[i][1][0] << 16));
                tr[i][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t *)(lds + 24576 + lane * 8 + i * 512));
                tr[i][1] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t *)(lds + 32768 + lane * 8 + i * 512));
            }
            if (MIX == 10 || MIX == 11) {
                x[(k + 1) & 7] = __builtin_amdgcn_exp2f(__builtin_fmaf(x[(k + 1) & 7], 1.0001f, -0.5f));
                x[(k + 2) & 7] += x[(k + 3) & 7];
            }
            if (MIX == 11 || MIX == 12) lb[i] = *(__attribute__((address_space(3))) uint4_t *)(lds + 8192 + addr + i * 1024);
            if (MIX == 12) {
                // a tile transposed once per workgroup instead of once per wavefront: this wavefront's share per step
                // (half a transposing read, a quarter of a 16-byte write of what such reads brought eight steps ago)
                if ((k & 1) == 0) tr[i][0] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t *)(lds + 24576 + lane * 8 + i * 512));
                if ((k & 3) == 3) {
                    const uint2_t u0 = __builtin_bit_cast(uint2_t, tr[(i + 1) & 7][0]), u1 = __builtin_bit_cast(uint2_t, tr[(i + 3) & 7][0]);
                    *(__attribute__((address_space(3))) uint4_t *)(lds + 32768 + addr + (k >> 2) * 1024) = uint4_t{u0[0], u0[1], u1[0], u1[1]};
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    float res = (float)sacc;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        res += x[i] + (float)la[i][0] + (float)lb[i][1] + (float)lc[i][2] + (float)tr[i][0][1] + (float)tr[i][1][2];
#pragma unroll
        for (int r = 0; r < 16; r++) res += acc[i][r];
    }
    const uint64_t c1 = clock64(), w1 = wall_clock64();
    sink[blockIdx.x * 256 + threadIdx.x] = res;
    if (threadIdx.x == 0) {
        ticks[2 * blockIdx.x] = c1 - c0;
        ticks[2 * blockIdx.x + 1] = w1 - w0;
    }
}

int launch_calibration_issue(int mix, int compute_units, int rounds, void *scratch, hipStream_t stream) {
    float *sink = (float *)scratch;
    uint64_t *ticks = (uint64_t *)((char *)scratch + (size_t)compute_units * 256 * sizeof(float));
    const dim3 grid((unsigned)compute_units);
#define FHIP_ISSUE(M) \
    case M: hipLaunchKernelGGL((issue_probe_kernel<M>), grid, dim3(256), 0, stream, sink, ticks, rounds); break
    switch (mix) {
        FHIP_ISSUE(0); FHIP_ISSUE(1); FHIP_ISSUE(2); FHIP_ISSUE(3); FHIP_ISSUE(4); FHIP_ISSUE(5);
        FHIP_ISSUE(6); FHIP_ISSUE(7); FHIP_ISSUE(8); FHIP_ISSUE(9); FHIP_ISSUE(10); FHIP_ISSUE(11); FHIP_ISSUE(12);
        default: set_error("calibration: mix %d is not one of 0..12", mix); return FHIP_ERR_INVALID_ARG;
    }
#undef FHIP_ISSUE
    FHIP_HIP_CHECK(hipGetLastError());
    return FHIP_OK;
}

size_t calibration_mfma_bytes(int compute_units) { return (size_t)compute_units * (256 * sizeof(float) + 2 * sizeof(uint64_t)); }

int launch_calibration_mfma(fhip_dtype dtype, int compute_units, int duty_percent, int rounds, int random_operands, void *scratch,
                            hipStream_t stream) {
    float *sink = (float *)scratch;
    uint64_t *ticks = (uint64_t *)((char *)scratch + (size_t)compute_units * 256 * sizeof(float));
    const int units = sleep_units(duty_percent);
    const dim3 grid((unsigned)compute_units);
    if (dtype == FHIP_F16) return launch_burn_t<half_t>(units, grid, stream, sink, ticks, rounds, random_operands);
    if (dtype == FHIP_BF16) return launch_burn_t<bf16_t>(units, grid, stream, sink, ticks, rounds, random_operands);
    set_error("calibration: the matrix-core loop takes f16 or bf16");
    return FHIP_ERR_UNSUPPORTED;
}

}  // namespace fhip
