// Probe: where do vector instructions hide under bf16 MFMAs on a CDNA4 SIMD?
// Eight waves per CU (two per SIMD) run loops of v_mfma_f32_32x32x16_bf16 and of
// independent f32 FMAs in four arrangements; the program prints the time per
// group of four MFMAs of a wave. Nothing in the library depends on it; its
// results are what the bf16 prefill kernel's hand-written instruction order
// (q8_gemm_bf16x3.hpp) rests on.
//
//   mode 0  every wave: MFMAs only                  (the matrix pipe's rate)
//   mode 4  one wave per SIMD: MFMAs only
//   mode 1  every wave: V FMAs per MFMA slot, no MFMAs
//   mode 2  one wave per SIMD MFMAs only, its partner wave FMAs only
//   mode 3  every wave: one MFMA, then V FMAs, repeated
//   mode 5  the same with one wave per SIMD
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
#define CHECK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); exit(1); } } while (0)

// mode 0: every wave MFMA only; 1: every wave VALU only; 2: waves 0-3 MFMA, 4-7 VALU;
// 3: every wave 1 MFMA + V valu interleaved; 4: waves 0-3 MFMA only (4-7 exit);
// 5: like 3 with one wave per SIMD (waves 4-7 exit)
template <int MODE, int V>
__global__ __launch_bounds__(512, 1) void k(float *out, int iters, float seed) {
    const int wave = threadIdx.x >> 6;
    floatx16_t acc[4];
    for (int c = 0; c < 4; ++c) for (int v = 0; v < 16; ++v) acc[c][v] = seed * v;
    float f[8];
    for (int i = 0; i < 8; ++i) f[i] = seed + i + threadIdx.x;
    bf16x8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed - i); }
    if (MODE == 5 && wave >= 4) {
        return;
    }
    const bool do_mfma = MODE == 0 || MODE == 3 || MODE == 5 || ((MODE == 2 || MODE == 4) && wave < 4);
    const bool do_valu = MODE == 1 || MODE == 3 || (MODE == 2 && wave >= 4);
    if (MODE == 3 || MODE == 5) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
#pragma unroll
                for (int i = 0; i < V; ++i) f[i % 8] = __builtin_fmaf(f[i % 8], 1.0001f, seed);
            }
        }
    } else if (do_mfma) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 4; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
        }
    } else if (do_valu) {
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
#pragma unroll
                for (int i = 0; i < V; ++i) f[i % 8] = __builtin_fmaf(f[i % 8], 1.0001f, seed);
            }
        }
    }
    float s = 0;
    for (int c = 0; c < 4; ++c) for (int v = 0; v < 16; ++v) s += acc[c][v];
    for (int i = 0; i < 8; ++i) s += f[i];
    if (s == 12345.678f) out[threadIdx.x] = s;
}

// CH accumulators per wave, used round-robin: CH = 1 is one chain of dependent
// MFMAs (each takes the one before as its C operand), CH = 4 four independent ones.
// WAVES = 4: one wave per SIMD (the other four exit), 8: two.
template <int CH, int WAVES>
__global__ __launch_bounds__(512, 1) void chains(float *out, int iters, float seed) {
    if ((int)(threadIdx.x >> 6) >= WAVES) {
        return;
    }
    floatx16_t acc[CH];
    for (int c = 0; c < CH; ++c) for (int v = 0; v < 16; ++v) acc[c][v] = seed * v;
    bf16x8_t a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (__bf16)(seed + i); b[i] = (__bf16)(seed - i); }
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            acc[m % CH] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[m % CH], 0, 0, 0);
        }
    }
    float s = 0;
    for (int c = 0; c < CH; ++c) for (int v = 0; v < 16; ++v) s += acc[c][v];
    if (s == 12345.678f) out[threadIdx.x] = s;
}

template <int CH, int WAVES> void run_chains(float *out) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    for (int w = 0; w < 2; ++w) chains<CH, WAVES><<<256, 512>>>(out, iters, 0.5f);
    CHECK(hipEventRecord(e0));
    chains<CH, WAVES><<<256, 512>>>(out, iters, 0.5f);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
    printf("%d wave(s) per SIMD, %d accumulator chain(s) per wave:   %8.1f us  %6.1f ns per 4 MFMAs of a wave\n",
           WAVES / 4, CH, ms * 1e3, ms * 1e6 / iters);
    fflush(stdout);
}

template <int MODE, int V> void run(const char *name, float *out) {
    const int iters = 20000;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0)); CHECK(hipEventCreate(&e1));
    for (int w = 0; w < 2; ++w) k<MODE, V><<<256, 512>>>(out, iters, 0.5f);
    CHECK(hipEventRecord(e0));
    k<MODE, V><<<256, 512>>>(out, iters, 0.5f);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms; CHECK(hipEventElapsedTime(&ms, e0, e1));
    printf("%-44s V=%2d  %8.1f us  %6.1f ns per 4-MFMA group\n", name, V, ms * 1e3, ms * 1e6 / iters);
    fflush(stdout);
}

int main() {
    float *out; CHECK(hipMalloc(&out, 4096));
    run<0, 0>("all 8 waves MFMA", out);
    run<4, 0>("4 waves MFMA (one per SIMD)", out);
    run<1, 8>("all 8 waves VALU", out);
    run<1, 16>("all 8 waves VALU", out);
    run<2, 8>("4 waves MFMA + 4 waves VALU", out);
    run<2, 16>("4 waves MFMA + 4 waves VALU", out);
    run<2, 32>("4 waves MFMA + 4 waves VALU", out);
    run<3, 2>("each wave MFMA + V VALU interleaved", out);
    run<3, 4>("each wave MFMA + V VALU interleaved", out);
    run<3, 6>("each wave MFMA + V VALU interleaved", out);
    run<3, 8>("each wave MFMA + V VALU interleaved", out);
    run<3, 16>("each wave MFMA + V VALU interleaved", out);
    run<5, 2>("one wave per SIMD: MFMA + V VALU interleaved", out);
    run<5, 4>("one wave per SIMD: MFMA + V VALU interleaved", out);
    run<5, 6>("one wave per SIMD: MFMA + V VALU interleaved", out);
    run<5, 8>("one wave per SIMD: MFMA + V VALU interleaved", out);
    run_chains<1, 4>(out);
    run_chains<2, 4>(out);
    run_chains<4, 4>(out);
    run_chains<1, 8>(out);
    run_chains<2, 8>(out);
    return 0;
}
