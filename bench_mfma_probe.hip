// What the matrix cores of the device at hand give a loop of nothing but matrix instructions: the
// denominator "measured on the box" beside the published peak that the benchmark prices against.
// Built by bench.py as a library of its own; nothing on the product path calls it.
//
// Role in the reference: none (its benchmarks report times only, docs/benchmark-protocol.md:43-75).
#include "common.cuh"

namespace ms {

// Every wave keeps ACC independent accumulators in turn so that its matrix instructions follow one
// another without waiting for a result; the operands stay in registers.  The sums go to `out` so that
// the loop is not optimised away.
constexpr int PROBE_ACC = 16;

__global__ __launch_bounds__(256) void mfma_probe_kernel(float* __restrict__ out, int iters) {
    Frag a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        a.v[i] = from_f32<elem_t>(0.001f * (float)((threadIdx.x + i) & 7));
        b.v[i] = from_f32<elem_t>(0.002f * (float)((threadIdx.x * 3 + i) & 7));
    }
    f32x4 acc[PROBE_ACC];
#pragma unroll
    for (int j = 0; j < PROBE_ACC; ++j) acc[j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < PROBE_ACC; ++j) mma_16x16x32(acc[j], a, b);
    }
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < PROBE_ACC; ++j) s += acc[j][0] + acc[j][1] + acc[j][2] + acc[j][3];
    out[(size_t)blockIdx.x * 256 + threadIdx.x] = s;
}

}  // namespace ms

using namespace ms;

// Launches `blocks` blocks of four waves that each run `iters` rounds of PROBE_ACC products of 16x16x32.
// `out` holds blocks * 256 floats.  Returns through *flops the floating-point operations of the launch.
extern "C" int ms_probe_mfma(float* out, int blocks, int iters, double* flops, hipStream_t stream) {
    MS_REQUIRE(out && blocks > 0 && iters > 0, "mfma probe: %d blocks, %d rounds", blocks, iters);
    hipLaunchKernelGGL(mfma_probe_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, out, iters);
    if (flops) *flops = (double)blocks * 4.0 * (double)iters * PROBE_ACC * (2.0 * 16 * 16 * 32);
    return check_launch("mfma_probe");
}
