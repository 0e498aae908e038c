/*
 * argmax.hip - index of the first largest logit, the greedy pick after the output projection.
 *
 * What the sequential loop `best = 0; for j in 1..n-1: if (v[j] > v[best]) best = j` returns
 * (server/server_llm.c:224-228, cpu/llm/test_transformer.c:298-301): the lowest index among the
 * largest values; a NaN is never picked unless it sits at index 0, in which case nothing beats it.
 * Two small launches: 256 workgroups each reduce one contiguous slice of the vector to a
 * candidate (a single compute unit pulling the whole vector, freshly written by all the others,
 * measured 50 us for 600 KB), then one workgroup merges the 256 candidates. The candidates live in
 * the caller's result buffer behind the 8 result bytes, so nothing is allocated and concurrent
 * calls with different result buffers do not meet. Every thread starts from element 0 and
 * candidates are merged with "larger value, then lower index", which does not depend on the order
 * of the merge.
 */
#include "../../include/qlinear.h"
#include "qlin_device.h"
#include "qlin_internal.h"

namespace qlin {

namespace {
struct Cand { float v; int i; };
/* true if b should replace a */
__device__ __forceinline__ bool better(const Cand &b, const Cand &a) {
    return b.v > a.v || (b.v == a.v && b.i < a.i);
}
}  // namespace

constexpr int kSlices = 256;  /* candidates of the first stage */
static_assert(8 + 8 * kSlices == QLIN_ARGMAX_RESULT_BYTES, "result buffer: 8 result bytes + one candidate per slice");

/* best over one wave, then over the waves of the workgroup; valid in thread 0 */
template <int WAVES>
__device__ __forceinline__ Cand workgroup_best(Cand best, Cand *per_wave) {
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const Cand o = {__shfl_xor(best.v, off, 64), __shfl_xor(best.i, off, 64)};
        if (better(o, best)) best = o;
    }
    if (lane == 0) per_wave[wv] = best;
    __syncthreads();
    if (threadIdx.x == 0)
        for (int w = 1; w < WAVES; w++)
            if (better(per_wave[w], best)) best = per_wave[w];
    return best;
}

/* VEC: v is 16-byte aligned and a slice is a multiple of 4 elements, so a thread takes four consecutive
 * elements per step with one load and all of a thread's loads can be in flight together (the vector was
 * written a moment ago by every compute unit of the chip: each load is a trip to memory, and a chain of
 * scalar loads per thread cost 15 us for 152 k logits). */
template <bool VEC>
__global__ void __launch_bounds__(256)
argmax_slices_kernel(const float *__restrict__ v, int n, int per, float *__restrict__ result) {
    __shared__ Cand per_wave[4];
    const int lo = blockIdx.x * per, hi = min(n, lo + per);
    Cand best = {v[0], 0};
    if (VEC) {
        for (int j = lo + 4 * (int)threadIdx.x; j < hi; j += 1024) {
            if (j + 4 <= hi) {
                const float4 q = *reinterpret_cast<const float4 *>(v + j);
                const float e[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
                for (int u = 0; u < 4; u++) { /* ascending index: a tie keeps the lower one */
                    const Cand c = {e[u], j + u};
                    if (better(c, best)) best = c;
                }
            } else {
                for (int u = j; u < hi; u++) {
                    const Cand c = {v[u], u};
                    if (better(c, best)) best = c;
                }
            }
        }
    } else {
        for (int j = lo + threadIdx.x; j < hi; j += 256) {
            const Cand c = {v[j], j};
            if (better(c, best)) best = c;
        }
    }
    best = workgroup_best<4>(best, per_wave);
    if (threadIdx.x == 0) {
        result[2 + 2 * blockIdx.x] = __int_as_float(best.i);
        result[3 + 2 * blockIdx.x] = best.v;
    }
}

__global__ void __launch_bounds__(256)
argmax_merge_kernel(float *__restrict__ result) {
    __shared__ Cand per_wave[4];
    Cand best = {result[3 + 2 * threadIdx.x], __float_as_int(result[2 + 2 * threadIdx.x])};
    best = workgroup_best<4>(best, per_wave);
    if (threadIdx.x == 0) {
        result[0] = __int_as_float(best.i);
        result[1] = best.v;
    }
}

hipError_t launch_argmax(const float *v, int n, float *result, hipStream_t stream) {
    const int per = (((n + kSlices - 1) / kSlices) + 3) & ~3; /* elements per slice, a multiple of 4 */
    if ((reinterpret_cast<uintptr_t>(v) & 15u) == 0)
        hipLaunchKernelGGL(argmax_slices_kernel<true>, dim3(kSlices), dim3(256), 0, stream, v, n, per, result);
    else
        hipLaunchKernelGGL(argmax_slices_kernel<false>, dim3(kSlices), dim3(256), 0, stream, v, n, per, result);
    hipLaunchKernelGGL(argmax_merge_kernel, dim3(1), dim3(256), 0, stream, result);
    return hipGetLastError();
}

}  // namespace qlin
