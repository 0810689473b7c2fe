// Opacity and scale of the copies when a Gaussian is split into n equal ones, equation (9) of
// "3D Gaussian Splatting as Markov Chain Monte Carlo"; follows
// gsplat/cuda/csrc/relocation.cu:4-30 of the reference, including its mixed precision (the
// powers and the square root are taken in double, the sum is kept in float).
#include "common.h"

namespace {

__global__ void __launch_bounds__(SPLATAD_THREADS)
compute_relocation_kernel(uint32_t N, const float *__restrict__ opacities,
                          const float *__restrict__ scales, const int32_t *__restrict__ ratios,
                          const float *__restrict__ binoms, int32_t n_max,
                          float *__restrict__ new_opacities, float *__restrict__ new_scales) {
    const uint32_t idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= N) return;
    const int32_t n = ratios[idx];
    const float o = opacities[idx];
    const float o_new = 1.0f - powf(1.0f - o, 1.0f / (float)n);
    new_opacities[idx] = o_new;
    float denom = 0.0f;
    for (int32_t i = 1; i <= n; ++i) {
        double power = (double)o_new; // o_new^(k+1)
        for (int32_t k = 0; k <= i - 1; ++k) {
            const float bin = binoms[(size_t)(i - 1) * n_max + k];
            const double sign = (k & 1) ? -1.0 : 1.0;
            const float term = (float)((sign / sqrt((double)(float)(k + 1))) * power);
            denom += bin * term;
            power *= (double)o_new;
        }
    }
    const float coeff = o / denom;
#pragma unroll
    for (int q = 0; q < 3; ++q) new_scales[(size_t)idx * 3 + q] = coeff * scales[(size_t)idx * 3 + q];
}

} // namespace

extern "C" int splatad_compute_relocation(uint32_t N, const float *opacities, const float *scales,
                                          const int32_t *ratios, const float *binoms,
                                          int32_t n_max, float *new_opacities, float *new_scales,
                                          splatad_stream_t stream) {
    if (N == 0) return 0;
    SPLATAD_REQUIRE(opacities && scales && ratios && binoms && new_opacities && new_scales,
                    "compute_relocation: null pointer argument");
    SPLATAD_REQUIRE(n_max >= 1, "compute_relocation: n_max is %d", n_max);
    hipLaunchKernelGGL(compute_relocation_kernel, dim3((N + SPLATAD_THREADS - 1) / SPLATAD_THREADS),
                       dim3(SPLATAD_THREADS), 0, (hipStream_t)stream, N, opacities, scales, ratios,
                       binoms, n_max, new_opacities, new_scales);
    SPLATAD_LAUNCH_CHECK();
    return 0;
}
