/*
 * moe.hip - MoE expert FFN pieces (common/transformer.h:4045-4131).
 *
 *   route:    softmax over all experts, keep the top_k largest, renormalise by their sum
 *             (:4054-4091). One wavefront per token. The k survivors are written in
 *             descending weight order (ties: lower expert index first); the reference's heap
 *             leaves them in heap order, which only changes the order of the final fp32 sum.
 *   silu_mul: h = gate/(1+exp(-gate)) * up (:4108, scalar form :4690)
 *   axpy:     out += w * q (:4116-4127)
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

__global__ void __launch_bounds__(64)
moe_route_kernel(const float *__restrict__ logits, int n_expert, int top_k, int32_t *__restrict__ idx,
                 float *__restrict__ wgt) {
    extern __shared__ float prob[]; /* n_expert floats */
    const int tok = blockIdx.x, lane = threadIdx.x;
    const float *lg = logits + (size_t)tok * n_expert;
    float mx = -INFINITY;
    for (int e = lane; e < n_expert; e += 64) mx = fmaxf(mx, lg[e]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.0f;
    for (int e = lane; e < n_expert; e += 64) {
        const float p = expf(lg[e] - mx);
        prob[e] = p;
        sum += p;
    }
    sum = wave_sum(sum);
    __syncthreads();
    for (int e = lane; e < n_expert; e += 64) prob[e] /= sum;
    __syncthreads();
    float wsum = 0.0f;
    for (int k = 0; k < top_k; k++) {
        /* arg-max over what is left: larger weight wins, then the lower index */
        float best = -1.0f;
        int bi = 0x7FFFFFFF;
        for (int e = lane; e < n_expert; e += 64) {
            const float p = prob[e];
            if (p > best) { best = p; bi = e; }
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const float ob = __shfl_xor(best, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        if (lane == 0) {
            idx[(size_t)tok * top_k + k] = bi;
            wgt[(size_t)tok * top_k + k] = best;
            prob[bi] = -2.0f;
        }
        wsum += best;
        __syncthreads();
    }
    if (wsum > 0.0f)
        for (int k = lane; k < top_k; k += 64) wgt[(size_t)tok * top_k + k] /= wsum;
}

__global__ void __launch_bounds__(256)
silu_mul_kernel(float *__restrict__ h, const float *__restrict__ gate, const float *__restrict__ up, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const float g = gate[i];
        h[i] = g / (1.0f + expf(-g)) * up[i];
    }
}

/* out[i] (+)= w[widx] * q[i]; the weight is read on the device so that the host never waits */
__global__ void __launch_bounds__(256)
axpy_dev_weight_kernel(float *__restrict__ out, const float *__restrict__ q, const float *__restrict__ w,
                       int widx, int n, int overwrite) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = (overwrite ? 0.0f : out[i]) + w[widx] * q[i];
}

hipError_t launch_moe_route(const float *logits, int n_tok, int n_expert, int top_k, int32_t *idx,
                            float *w, hipStream_t s) {
    if (n_tok == 0) return hipSuccess;
    hipLaunchKernelGGL(moe_route_kernel, dim3(n_tok), dim3(64), (size_t)n_expert * sizeof(float), s,
                       logits, n_expert, top_k, idx, w);
    return hipGetLastError();
}

hipError_t launch_silu_mul(float *h, const float *gate, const float *up, int n, hipStream_t s) {
    hipLaunchKernelGGL(silu_mul_kernel, dim3((n + 255) / 256), dim3(256), 0, s, h, gate, up, n);
    return hipGetLastError();
}

hipError_t launch_axpy_dev_weight(float *out, const float *q, const float *w, int widx, int n,
                                  int overwrite, hipStream_t s) {
    hipLaunchKernelGGL(axpy_dev_weight_kernel, dim3((n + 255) / 256), dim3(256), 0, s, out, q, w, widx, n,
                       overwrite);
    return hipGetLastError();
}

}  // namespace qlin
