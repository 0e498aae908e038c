/*
 * moe.hip - MoE expert FFN pieces (common/transformer.h:4045-4131).
 *
 *   route:    softmax over all experts, keep the top_k largest, renormalise by their sum
 *             (:4054-4091). One wavefront per token. The k survivors are written in
 *             descending weight order; the reference's heap leaves them in heap order, which only
 *             changes the order of the final fp32 sum. Where the choice itself depends on the heap -
 *             the k-th and (k+1)-th largest probabilities are equal, or probabilities are NaN - one
 *             lane replays the reference's min-heap literally (:4057-4091), so the SET of experts
 *             and their weights are the reference's in every case.
 *   silu_mul: h = gate/(1+exp(-gate)) * up (:4108, scalar form :4690)
 *   axpy:     out += w * q (:4116-4127)
 */
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

/* the reference's selection, statement for statement (common/transformer.h:4057-4091): a min-heap of the
 * top_k largest so far over one pass, then the weights divided by their sum. One lane; heap in idx/w. */
__device__ void route_heap(const float *prob, int n_expert, int top_k, int32_t *idx, float *w) {
    int k = 0;
    for (int e = 0; e < n_expert; e++) {
        const float pe = prob[e];
        if (k < top_k) {
            idx[k] = e;
            w[k] = pe;
            k++;
            for (int j = k - 1; j > 0;) {
                const int parent = (j - 1) / 2;
                if (w[j] < w[parent]) {
                    const float tv = w[j]; w[j] = w[parent]; w[parent] = tv;
                    const int ti = idx[j]; idx[j] = idx[parent]; idx[parent] = ti;
                    j = parent;
                } else break;
            }
        } else if (pe > w[0]) {
            w[0] = pe;
            idx[0] = e;
            for (int j = 0;;) {
                int s = j;
                const int l = 2 * j + 1, r = 2 * j + 2;
                if (l < top_k && w[l] < w[s]) s = l;
                if (r < top_k && w[r] < w[s]) s = r;
                if (s == j) break;
                const float tv = w[j]; w[j] = w[s]; w[s] = tv;
                const int ti = idx[j]; idx[j] = idx[s]; idx[s] = ti;
                j = s;
            }
        }
    }
    float wsum = 0.0f;
    for (int i = 0; i < top_k; i++) wsum += w[i];
    if (wsum > 0.0f)
        for (int i = 0; i < top_k; i++) w[i] /= wsum;
}

/* Probabilities live in registers, PL per lane (expert e = lane + 64 j); every selection step is one
 * wave maximum on the cross-lane data path plus a ballot for the lowest expert index holding it. The
 * general form (more than 64 * 8 experts) keeps them in LDS and reads them back per step. */
template <int PL>
__global__ void __launch_bounds__(64)
moe_route_kernel(const float *__restrict__ logits, int n_expert, int top_k, int32_t *__restrict__ idx,
                 float *__restrict__ wgt) {
    const int tok = blockIdx.x, lane = threadIdx.x;
    const float *lg = logits + (size_t)tok * n_expert;
    float p[PL];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < PL; j++) {
        const int e = lane + 64 * j;
        p[j] = e < n_expert ? lg[e] : -INFINITY;
        mx = fmaxf(mx, p[j]);
    }
    mx = wave_max_dpp(mx);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < PL; j++) {
        const int e = lane + 64 * j;
        p[j] = e < n_expert ? expf(p[j] - mx) : -1.0f; /* empty slots never win */
        sum += e < n_expert ? p[j] : 0.0f;
    }
    sum = wave_sum_dpp(sum);
    __shared__ float prob_copy[64 * PL];
#pragma unroll
    for (int j = 0; j < PL; j++) {
        if (lane + 64 * j < n_expert) p[j] /= sum;
        prob_copy[lane + 64 * j] = p[j];
    }
    float wsum = 0.0f, mine = 0.0f; /* lane k keeps the k-th weight (top_k <= 64) */
    int mine_idx = 0;
    bool replay = false; /* the heap decides: a pick found nothing (NaN), or the last pick ties with what is left */
    float last = 0.0f;
    for (int k = 0; k < top_k; k++) {
        float best = -1.0f;
#pragma unroll
        for (int j = 0; j < PL; j++) best = fmaxf(best, p[j]);
        best = wave_max_dpp(best);
        /* the lowest expert index among those that hold the maximum: slots j in order, lowest lane first */
        int bi = 0x7FFFFFFF;
#pragma unroll
        for (int j = 0; j < PL; j++) {
            const unsigned long long m = __ballot(p[j] == best);
            if (bi == 0x7FFFFFFF && m != 0ull) bi = __builtin_ctzll(m) + 64 * j;
        }
        if (bi >= n_expert) { bi = 0; best = 0.0f; replay = true; } /* NaN probabilities compare false everywhere */
#pragma unroll
        for (int j = 0; j < PL; j++)
            if (lane + 64 * j == bi) p[j] = -2.0f;
        if (lane == k) { mine = best; mine_idx = bi; }
        wsum += best;
        last = best;
    }
    {
        float rest = -1.0f;
#pragma unroll
        for (int j = 0; j < PL; j++) rest = fmaxf(rest, p[j]);
        rest = wave_max_dpp(rest);
        if (top_k < n_expert && rest == last) replay = true;
    }
    if (replay) { /* uniform: every lane holds the same flags */
        __syncthreads();
        if (lane == 0) route_heap(prob_copy, n_expert, top_k, idx + (size_t)tok * top_k, wgt + (size_t)tok * top_k);
        return;
    }
    if (lane < top_k) {
        idx[(size_t)tok * top_k + lane] = mine_idx;
        wgt[(size_t)tok * top_k + lane] = wsum > 0.0f ? mine / wsum : mine;
    }
}

__global__ void __launch_bounds__(64)
moe_route_lds_kernel(const float *__restrict__ logits, int n_expert, int top_k, int32_t *__restrict__ idx,
                     float *__restrict__ wgt) {
    extern __shared__ float prob[]; /* n_expert floats */
    const int tok = blockIdx.x, lane = threadIdx.x;
    const float *lg = logits + (size_t)tok * n_expert;
    float mx = -INFINITY;
    for (int e = lane; e < n_expert; e += 64) mx = fmaxf(mx, lg[e]);
    mx = wave_max_dpp(mx);
    float sum = 0.0f;
    for (int e = lane; e < n_expert; e += 64) {
        const float p = expf(lg[e] - mx);
        prob[e] = p;
        sum += p;
    }
    sum = wave_sum_dpp(sum);
    __syncthreads();
    for (int e = lane; e < n_expert; e += 64) prob[e] /= sum;
    __syncthreads();
    float wsum = 0.0f, last = 0.0f;
    bool replay = false;
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
        if (bi >= n_expert) { replay = true; break; } /* NaN probabilities compare false everywhere */
        if (lane == 0) {
            idx[(size_t)tok * top_k + k] = bi;
            wgt[(size_t)tok * top_k + k] = best;
            prob[bi] = -2.0f - (float)k; /* marks pick k; undone below if the heap has to decide */
        }
        wsum += best;
        last = best;
        __syncthreads();
    }
    if (!replay && top_k < n_expert) { /* does the last pick tie with what is left? */
        float rest = -1.0f;
        for (int e = lane; e < n_expert; e += 64) rest = fmaxf(rest, prob[e]);
        rest = wave_max_dpp(rest);
        replay = rest == last;
    }
    if (replay) { /* uniform; put the picked probabilities back and replay the reference's heap */
        __syncthreads();
        if (lane == 0) {
            for (int e = 0; e < n_expert; e++)
                if (prob[e] <= -2.0f) prob[e] = wgt[(size_t)tok * top_k + (int)(-2.0f - prob[e])];
            route_heap(prob, n_expert, top_k, idx + (size_t)tok * top_k, wgt + (size_t)tok * top_k);
        }
        return;
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
    if (top_k <= 64 && n_expert <= 64 * 8) {
        if (n_expert <= 64)
            hipLaunchKernelGGL(moe_route_kernel<1>, dim3(n_tok), dim3(64), 0, s, logits, n_expert, top_k, idx, w);
        else if (n_expert <= 128)
            hipLaunchKernelGGL(moe_route_kernel<2>, dim3(n_tok), dim3(64), 0, s, logits, n_expert, top_k, idx, w);
        else if (n_expert <= 256)
            hipLaunchKernelGGL(moe_route_kernel<4>, dim3(n_tok), dim3(64), 0, s, logits, n_expert, top_k, idx, w);
        else
            hipLaunchKernelGGL(moe_route_kernel<8>, dim3(n_tok), dim3(64), 0, s, logits, n_expert, top_k, idx, w);
    } else {
        hipLaunchKernelGGL(moe_route_lds_kernel, dim3(n_tok), dim3(64), (size_t)n_expert * sizeof(float), s,
                           logits, n_expert, top_k, idx, w);
    }
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
