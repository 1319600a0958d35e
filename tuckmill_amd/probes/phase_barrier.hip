// phase_barrier.hip — what a dependent phase boundary costs INSIDE one persistent
// kernel on MI355X, to set beside what it costs as a kernel boundary.
//
// The decode step of a transformer is a chain of dependent phases (norm + q,k,v
// -> o + residual -> norm + gate,up + activation -> down + residual; 113 phases
// for 28 layers and the vocabulary projection), each streaming a few megabytes
// of weights. Issued as one kernel launch per phase the step is bound by the
// 5-6 us a dependent launch lasts (crates/tuckcore/src/engine/metal.rs:496-511,
// :1125-1131 issue the same chain per token). The alternative measured here: one
// launch for the whole chain, as many workgroups as stay resident, tiles
// assigned statically, every phase boundary a barrier across all workgroups
// built from plain device-scope stores (one flag per workgroup) that wave 0 of
// every workgroup polls with wave-wide device-scope loads; the first weight load
// of the next phase is issued before the wait. Every wait is bounded (it gives
// up and flags an error), so the kernel always exits.
//
// Build: hipcc --offload-arch=gfx950 -O2 -o phase_barrier phase_barrier.hip
// (tuckmill_amd/build.py does). Prints microseconds per phase for several
// phase sizes and grid sizes. A measurement probe: nothing in the library calls it.
#include <hip/hip_runtime.h>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <vector>
typedef unsigned u4 __attribute__((ext_vector_type(4)));
struct Args { unsigned P, T, rows_per_tile, cols; const unsigned char *w; float *v0, *v1; unsigned *flags, *err; unsigned spin_limit, epoch; };
__global__ __launch_bounds__(256) void chain(const Args a) {
    const unsigned lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const unsigned G = gridDim.x, wg = blockIdx.x;
    const unsigned gw = wg * 4u + wave, nw = G * 4u;
    __shared__ unsigned gave_up;
    if (threadIdx.x == 0) gave_up = 0;
    __syncthreads();
    for (unsigned p = 0; p < a.P; ++p) {
        // this wave's tiles of the phase: gw, gw + nw, ...
        unsigned tile = gw;
        const unsigned char *wt = a.w + ((size_t)(p % 8) * a.T + (tile < a.T ? tile : 0)) * a.rows_per_tile * a.cols;
        u4 q = __builtin_nontemporal_load((const u4 *)(wt + lane * 16u)); // prefetch before the wait
        if (p > 0) {
            if (wave == 0) {
                const unsigned want = a.epoch + p; // every flag >= want: phase p-1 complete everywhere
                unsigned spins = 0;
                for (;;) {
                    bool ok = true;
                    for (unsigned i = lane; i < G; i += 64u) {
                        ok = ok && (int)(__hip_atomic_load(a.flags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - want) >= 0;
                    }
                    if (__all(ok)) break;
                    if (++spins > a.spin_limit) { if (lane == 0) { *a.err = 1; gave_up = 1; } break; }
                    __builtin_amdgcn_s_sleep(2);
                }
            }
            __syncthreads();
        }
        const float *vin = (p & 1) ? a.v1 : a.v0;
        float *vout = (p & 1) ? a.v0 : a.v1;
        for (; tile < a.T; tile += nw) {
            float x[4];
            for (int i = 0; i < 4; ++i) x[i] = __hip_atomic_load(vin + lane * 4 + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            float acc = 0.f;
            wt = a.w + ((size_t)(p % 8) * a.T + tile) * a.rows_per_tile * a.cols;
            if (tile != gw) q = __builtin_nontemporal_load((const u4 *)(wt + lane * 16u));
            for (unsigned r = 0; r < a.rows_per_tile; ++r) {
                for (unsigned c = 0; c < a.cols; c += 1024u) {
                    acc += (float)(q.x & 0xff) * x[0] + (float)(q.y & 0xff) * x[1] + (float)(q.z & 0xff) * x[2] + (float)(q.w & 0xff) * x[3];
                    const unsigned rn = (c + 1024u < a.cols) ? r : r + 1, cn = (c + 1024u < a.cols) ? c + 1024u : 0;
                    if (rn < a.rows_per_tile) q = __builtin_nontemporal_load((const u4 *)(wt + (size_t)rn * a.cols + cn + lane * 16u));
                }
            }
            for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o, 64);
            if (lane == 0) __hip_atomic_store(vout + (tile % 256), acc * 1e-9f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8)); // this wave's stores are out
        __syncthreads();
        if (threadIdx.x == 0) __hip_atomic_store(a.flags + wg, a.epoch + p + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}
int main(int argc, char **argv) {
    const unsigned P = 113, cols = 1024;
    hipStream_t st; (void)hipStreamCreateWithFlags(&st, hipStreamNonBlocking);
    unsigned char *w; float *v0, *v1; unsigned *flags, *err;
    const size_t wbytes = (size_t)8 * 1024 * 8 * 1024 * 4;
    (void)hipMalloc(&w, wbytes); (void)hipMemset(w, 1, wbytes);
    (void)hipMalloc(&v0, 4096); (void)hipMalloc(&v1, 4096); (void)hipMemset(v0, 0, 4096); (void)hipMemset(v1, 0, 4096);
    (void)hipMalloc(&flags, 8192); (void)hipMalloc(&err, 4);
    (void)hipMemset(err, 0, 4); (void)hipMemset(flags, 0, 8192);
    unsigned epoch = 0;
    for (unsigned T : {128u, 256u, 512u, 1024u, 2048u}) for (unsigned rpt : {1u, 8u}) for (unsigned wgs : {128u, 256u, 512u}) {
        double best = 1e9;
        for (int rep = 0; rep < 5; ++rep) {
            Args a{P, T, rpt, cols, w, v0, v1, flags, err, 1u << 20, epoch};
            epoch += P + 1;
            (void)hipStreamSynchronize(st);
            auto t0 = std::chrono::steady_clock::now();
            hipLaunchKernelGGL(chain, dim3(wgs), dim3(256), 0, st, a);
            (void)hipStreamSynchronize(st);
            auto t1 = std::chrono::steady_clock::now();
            double us = std::chrono::duration<double, std::micro>(t1 - t0).count();
            best = us < best ? us : best;
        }
        unsigned e = 0; (void)hipMemcpy(&e, err, 4, hipMemcpyDeviceToHost);
        printf("T=%4u tiles/phase rows/tile=%u wgs=%4u: %8.1f us for %u phases = %.2f us/phase (%.1f MB/phase) err=%u\n", T, rpt, wgs, best, P, best / P, T * rpt * cols / 1e6, e);
    }
    return 0;
}
