/*
 * qlin_device.h - device-side view of the GGML block formats (gfx950).
 *
 * Byte layouts follow the packed block structs of common/ggml_dequant.h:30-204. Blocks are
 * addressed as raw bytes: inside a row only 2-byte alignment holds (block sizes 34, 210, 66,
 * 110 and 18 are not multiples of 4), so multi-byte fields are assembled from 16-bit loads
 * (the 17-byte MXFP4 block has byte fields only).
 */
#ifndef QLIN_DEVICE_H
#define QLIN_DEVICE_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qlin_codebooks.h"
#include "qlin_codebooks_ext.h"

namespace qlin {

enum : uint32_t {
    T_F32 = 0, T_F16 = 1, T_Q8_0 = 8, T_Q4_K = 12, T_Q5_K = 13, T_Q6_K = 14,
    T_IQ2_XXS = 16, T_IQ4_NL = 20, T_IQ3_S = 21, T_BF16 = 30,
    T_Q4_0 = 2, T_Q4_1 = 3, T_Q5_0 = 6, T_Q5_1 = 7, T_Q2_K = 10, T_Q3_K = 11, T_IQ2_XS = 17,
    T_IQ3_XXS = 18, T_IQ1_S = 19, T_IQ2_S = 22, T_IQ4_XS = 23, T_IQ1_M = 29, T_TQ1_0 = 34,
    T_TQ2_0 = 35, T_MXFP4 = 39, T_NVFP4 = 40, T_Q1_0 = 41
};

/* every block format with a decoder, for the type switches: X(type id) */
#define QLIN_FOR_EACH_BLOCK_TYPE(X)                                                              \
    X(T_Q8_0) X(T_Q4_K) X(T_Q5_K) X(T_Q6_K) X(T_IQ2_XXS) X(T_IQ4_NL) X(T_IQ3_S) X(T_Q4_0)       \
    X(T_Q4_1) X(T_Q5_0) X(T_Q5_1) X(T_Q2_K) X(T_Q3_K) X(T_IQ2_XS) X(T_IQ3_XXS) X(T_IQ1_S)      \
    X(T_IQ2_S) X(T_IQ4_XS) X(T_IQ1_M) X(T_TQ1_0) X(T_TQ2_0) X(T_MXFP4) X(T_NVFP4) X(T_Q1_0)

/* elements and bytes per block (common/ggml_dequant.h:261-294) */
template <uint32_t T> struct Geom;
template <> struct Geom<T_Q8_0>    { static constexpr int BE = 32,  BB = 34;  };
template <> struct Geom<T_Q4_K>    { static constexpr int BE = 256, BB = 144; };
template <> struct Geom<T_Q5_K>    { static constexpr int BE = 256, BB = 176; };
template <> struct Geom<T_Q6_K>    { static constexpr int BE = 256, BB = 210; };
template <> struct Geom<T_IQ2_XXS> { static constexpr int BE = 256, BB = 66;  };
template <> struct Geom<T_IQ4_NL>  { static constexpr int BE = 32,  BB = 18;  };
template <> struct Geom<T_IQ3_S>   { static constexpr int BE = 256, BB = 110; };

__host__ __device__ inline bool type_geometry(uint32_t t, int *be, int *bb) {
    switch (t) {
    case T_F32: *be = 1; *bb = 4; return true;
    case T_F16: case T_BF16: *be = 1; *bb = 2; return true;
    case T_Q8_0: *be = 32; *bb = 34; return true;
    case T_Q4_K: *be = 256; *bb = 144; return true;
    case T_Q5_K: *be = 256; *bb = 176; return true;
    case T_Q6_K: *be = 256; *bb = 210; return true;
    case T_IQ2_XXS: *be = 256; *bb = 66; return true;
    case T_IQ4_NL: *be = 32; *bb = 18; return true;
    case T_IQ3_S: *be = 256; *bb = 110; return true;
    case T_Q4_0: *be = 32; *bb = 18; return true;
    case T_Q4_1: *be = 32; *bb = 20; return true;
    case T_Q5_0: *be = 32; *bb = 22; return true;
    case T_Q5_1: *be = 32; *bb = 24; return true;
    case T_Q2_K: *be = 256; *bb = 84; return true;
    case T_Q3_K: *be = 256; *bb = 110; return true;
    case T_IQ2_XS: *be = 256; *bb = 74; return true;
    case T_IQ3_XXS: *be = 256; *bb = 98; return true;
    case T_IQ1_S: *be = 256; *bb = 50; return true;
    case T_IQ2_S: *be = 256; *bb = 82; return true;
    case T_IQ4_XS: *be = 256; *bb = 136; return true;
    case T_IQ1_M: *be = 256; *bb = 56; return true;
    case T_TQ1_0: *be = 256; *bb = 54; return true;
    case T_TQ2_0: *be = 256; *bb = 66; return true;
    case T_MXFP4: *be = 32; *bb = 17; return true;
    case T_NVFP4: *be = 64; *bb = 36; return true;
    case T_Q1_0: *be = 128; *bb = 18; return true;
    default: return false;
    }
}

__device__ __forceinline__ uint32_t ld_u16(const uint8_t *p) {
    return *reinterpret_cast<const uint16_t *>(p);
}
__device__ __forceinline__ uint32_t ld_u32_a2(const uint8_t *p) { /* 2-byte aligned dword */
    return ld_u16(p) | (ld_u16(p + 2) << 16);
}

/* hardware conversion: exact for every finite input (subnormals included) and for infinities;
 * quiets a signalling NaN */
__device__ __forceinline__ float half_bits_fast(uint32_t h) {
    union { unsigned short u; _Float16 f; } v;
    v.u = (unsigned short)h;
    return (float)v.f;
}

/* IEEE half -> float, bit-exact for every input like common/ggml_dequant.h:206-229, whose NaN
 * payloads pass through unquieted: the hardware conversion, with the bits of a NaN rebuilt by
 * hand. Written without a branch on the loaded value, so that the loads of several blocks can be
 * in flight before the first conversion. */
__device__ __forceinline__ float half_bits_exact(uint32_t h) {
    const float f = half_bits_fast(h);
    const uint32_t nan_bits = ((h & 0x8000u) << 16) | 0x7F800000u | ((h & 1023u) << 13);
    return (h & 0x7FFFu) > 0x7C00u ? __uint_as_float(nan_bits) : f;
}

/* sign byte of the 2/3-bit i-quants: 7 stored bits + their parity in bit 7
 * (table at common/ggml_dequant.h:1765-1774) */
__device__ __forceinline__ uint32_t iq_sign_byte(uint32_t i7) {
    return i7 | ((__popc(i7) & 1u) << 7);
}

/* 6-bit scale and min of sub-block g from the 12 packed bytes of a Q4_K/Q5_K super-block
 * (get_scale_min_k4, common/ggml_dequant.h:1582-1590) */
__device__ __forceinline__ void k4_scale_min(const uint8_t *s, int g, uint32_t &sc, uint32_t &mn) {
    if (g < 4) {
        sc = s[g] & 63u;
        mn = s[g + 4] & 63u;
    } else {
        sc = (s[g + 4] & 15u) | ((uint32_t)(s[g - 4] >> 6) << 4);
        mn = ((uint32_t)s[g + 4] >> 4) | ((uint32_t)(s[g] >> 6) << 4);
    }
}

/*
 * decode8<T>(blk, k0, y): elements k0..k0+7 (k0 a multiple of 8) of one block, with exactly
 * the reference's fp32 operation order, so that results are bit-identical:
 *   Q8_0     d*q                               common/ggml_dequant.h:1479-1489
 *   Q4_K/5_K (d*sc)*q - (dmin*m)               :1592-1651   (d*sc, dmin*m, (d*sc)*q are exact
 *                                              in fp32, so a fused multiply-subtract rounds the
 *                                              same way as the separate multiply and subtract)
 *   Q6_K     (d*sc)*q                          :1653-1687
 *   IQ4_NL   d*codebook[nibble]                :2942-2954
 *   IQ2_XXS  ((d*(0.5+s))*0.25)*grid*(+-1)     :2793-2816
 *   IQ3_S    (d*(1+2s))*grid*(+-1)             :3022-3058
 */
template <uint32_t T> struct Codec;

template <> struct Codec<T_Q8_0> : Geom<T_Q8_0> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int8_t *q = reinterpret_cast<const int8_t *>(blk + 2 + k0);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = d * (float)q[i];
    }
};

template <> struct Codec<T_Q4_K> : Geom<T_Q4_K> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const float dmin = half_bits_exact(ld_u16(blk + 2));
        const int g = k0 >> 5, l0 = k0 & 31;
        uint32_t sc, mn;
        k4_scale_min(blk + 4, g, sc, mn);
        const float dl = d * (float)sc, ml = dmin * (float)mn;
        const uint8_t *q = blk + 16 + (g >> 1) * 32 + l0;
        const int sh = (g & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = dl * (float)((q[i] >> sh) & 15) - ml;
    }
};

template <> struct Codec<T_Q5_K> : Geom<T_Q5_K> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const float dmin = half_bits_exact(ld_u16(blk + 2));
        const int g = k0 >> 5, l0 = k0 & 31;
        uint32_t sc, mn;
        k4_scale_min(blk + 4, g, sc, mn);
        const float dl = d * (float)sc, ml = dmin * (float)mn;
        const uint8_t *qh = blk + 16 + l0;
        const uint8_t *q = blk + 48 + (g >> 1) * 32 + l0;
        const int sh = (g & 1) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int v = ((q[i] >> sh) & 15) + (((qh[i] >> g) & 1) << 4);
            y[i] = dl * (float)v - ml;
        }
    }
};

template <> struct Codec<T_Q6_K> : Geom<T_Q6_K> {
    /* four codes at a time: the low nibbles and the two high bits are combined bytewise into q + 32
     * (0..63); (float)byte - 32.0f is exact and equals (float)(q), so dl * that rounds like the
     * reference's d * sc * q. */
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk + 208));
        const int half = k0 >> 7, r = k0 & 127, seg = r >> 5, l0 = r & 31;
        const uint8_t *ql = blk + 64 * half + 32 * (seg & 1) + l0;
        const uint8_t *qh = blk + 128 + 32 * half + l0;
        const int8_t sc = reinterpret_cast<const int8_t *>(blk + 192)[8 * half + 2 * seg + (l0 >> 4)];
        const float dl = d * (float)sc;
        const int nsh = (seg >> 1) * 4, hsh = 2 * seg;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const uint32_t lo = ld_u32_a2(ql + 4 * j), hi = ld_u32_a2(qh + 4 * j);
            const uint32_t q4 = ((lo >> nsh) & 0x0F0F0F0Fu) | (((hi >> hsh) & 0x03030303u) << 4);
#pragma unroll
            for (int i = 0; i < 4; i++) y[4 * j + i] = dl * ((float)((q4 >> (8 * i)) & 255u) - 32.0f);
        }
    }
};

template <> struct Codec<T_IQ4_NL> : Geom<T_IQ4_NL> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const uint8_t *q = blk + 2 + (k0 & 15);
        const int sh = (k0 >> 4) * 4;
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = d * (float)qlin_iq4nl_values[(q[i] >> sh) & 15];
    }
};

template <> struct Codec<T_IQ2_XXS> : Geom<T_IQ2_XXS> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t a0 = ld_u32_a2(blk + 2 + 8 * g), a1 = ld_u32_a2(blk + 6 + 8 * g);
        const float db = d * (0.5f + (float)(a1 >> 28)) * 0.25f;
        const uint64_t cell = qlin_iq2xxs_grid[(a0 >> (8 * l)) & 255u];
        const uint32_t sg = iq_sign_byte((a1 >> (7 * l)) & 127u);
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float mag = db * (float)(uint32_t)((cell >> (8 * i)) & 255u);
            y[i] = mag * (((sg >> i) & 1u) ? -1.0f : 1.0f);
        }
    }
};

template <> struct Codec<T_IQ3_S> : Geom<T_IQ3_S> {
    __device__ static void decode8(const uint8_t *blk, int k0, float (&y)[8]) {
        const float d = half_bits_exact(ld_u16(blk));
        const int g = k0 >> 5, l = (k0 & 31) >> 3;
        const uint32_t nib = (blk[106 + (g >> 1)] >> (4 * (g & 1))) & 15u;
        const float db = d * (float)(1u + 2u * nib);
        const uint32_t qh = blk[66 + g];
        const uint32_t i0 = blk[2 + 8 * g + 2 * l] | (((qh >> (2 * l)) & 1u) << 8);
        const uint32_t i1 = blk[2 + 8 * g + 2 * l + 1] | (((qh >> (2 * l + 1)) & 1u) << 8);
        const uint32_t c0 = qlin_iq3s_grid[i0], c1 = qlin_iq3s_grid[i1];
        const uint32_t sb = blk[74 + 4 * g + l];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float m0 = db * (float)((c0 >> (8 * i)) & 255u);
            const float m1 = db * (float)((c1 >> (8 * i)) & 255u);
            y[i] = m0 * (((sb >> i) & 1u) ? -1.0f : 1.0f);
            y[i + 4] = m1 * (((sb >> (i + 4)) & 1u) ? -1.0f : 1.0f);
        }
    }
};

/* Dense rows (F16, BF16, F32) seen by the matvec kernels as "blocks" of eight elements, so that
 * they run through the same row loops: what tf_qmatvec computes for these types is the fp32 dot of
 * the widened row with x (common/transformer.h:1051-1075, common/ggml_dequant.h:360-400, :1201-1230).
 * type_geometry() keeps the per-element view (1 element, 2 or 4 bytes) for the codec entry points. */
#define QLIN_FOR_EACH_DENSE_TYPE(X) X(T_F16) X(T_BF16) X(T_F32)
template <> struct Geom<T_F16>  { static constexpr int BE = 8, BB = 16; };
template <> struct Geom<T_BF16> { static constexpr int BE = 8, BB = 16; };
template <> struct Geom<T_F32>  { static constexpr int BE = 8, BB = 32; };

template <> struct Codec<T_F16> : Geom<T_F16> {
    __device__ static void decode8(const uint8_t *blk, int, float (&y)[8]) {
        const uint4 v = *reinterpret_cast<const uint4 *>(blk);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            y[2 * i] = half_bits_exact(w[i] & 0xFFFFu);
            y[2 * i + 1] = half_bits_exact(w[i] >> 16);
        }
    }
};
template <> struct Codec<T_BF16> : Geom<T_BF16> {
    __device__ static void decode8(const uint8_t *blk, int, float (&y)[8]) {
        const uint4 v = *reinterpret_cast<const uint4 *>(blk);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            y[2 * i] = __uint_as_float(w[i] << 16);
            y[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
        }
    }
};
template <> struct Codec<T_F32> : Geom<T_F32> {
    __device__ static void decode8(const uint8_t *blk, int, float (&y)[8]) {
        const float4 a = reinterpret_cast<const float4 *>(blk)[0], b = reinterpret_cast<const float4 *>(blk)[1];
        y[0] = a.x; y[1] = a.y; y[2] = a.z; y[3] = a.w; y[4] = b.x; y[5] = b.y; y[6] = b.z; y[7] = b.w;
    }
};

}  // namespace qlin
#include "qlin_codecs_ext.h"
namespace qlin {

/* wait until at most n vector-memory operations of this wavefront are outstanding (they retire
 * in order, so the oldest ones are then complete); n is wave-uniform, 0..15 (more waits for 15) */
__device__ __forceinline__ void wait_vm_at_most(int n) {
    switch (n) {
    case 0: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    case 1: asm volatile("s_waitcnt vmcnt(1)" ::: "memory"); break;
    case 2: asm volatile("s_waitcnt vmcnt(2)" ::: "memory"); break;
    case 3: asm volatile("s_waitcnt vmcnt(3)" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)" ::: "memory"); break;
    case 5: asm volatile("s_waitcnt vmcnt(5)" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)" ::: "memory"); break;
    case 7: asm volatile("s_waitcnt vmcnt(7)" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); break;
    case 9: asm volatile("s_waitcnt vmcnt(9)" ::: "memory"); break;
    case 10: asm volatile("s_waitcnt vmcnt(10)" ::: "memory"); break;
    case 11: asm volatile("s_waitcnt vmcnt(11)" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)" ::: "memory"); break;
    case 13: asm volatile("s_waitcnt vmcnt(13)" ::: "memory"); break;
    case 14: asm volatile("s_waitcnt vmcnt(14)" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(15)" ::: "memory"); break;
    }
}

template <int CTRL> __device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
/* sum over the 64 lanes with cross-lane data-path moves (no LDS round trips); uniform result */
__device__ __forceinline__ float wave_sum_dpp(float v) {
    v += dpp_mov<0xB1>(v);  /* quad_perm [1,0,3,2] */
    v += dpp_mov<0x4E>(v);  /* quad_perm [2,3,0,1] */
    v += dpp_mov<0x141>(v); /* row_half_mirror */
    v += dpp_mov<0x140>(v); /* row_mirror: every lane of a 16-lane row now holds the row total */
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

/* maximum over the 64 lanes, same moves; uniform result. NaN inputs are ignored (fmaxf). */
__device__ __forceinline__ float wave_max_dpp(float v) {
    v = fmaxf(v, dpp_mov<0xB1>(v));
    v = fmaxf(v, dpp_mov<0x4E>(v));
    v = fmaxf(v, dpp_mov<0x141>(v));
    v = fmaxf(v, dpp_mov<0x140>(v));
    return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}

/* Kernel-side view of one fused matvec launch: up to three matrices of one block type that share
 * x (host-side GemvJob, flattened so that nothing is indexed dynamically). mode 0: y = W.x,
 * 1: y += W.x, 2: y0 = silu(W0.x) * (W1.x) with n0 == n1. */
struct JobView {
    const uint8_t *W0, *W1, *W2;
    float *y0, *y1, *y2;
    int n0, n1, n2;
    int mode;
};
/* matrix and row of virtual row v, the rows of the matrices taken one after the other */
__device__ __forceinline__ void job_locate(const JobView &j, int v, const uint8_t *&W, float *&y, int &r) {
    if (v < j.n0) { W = j.W0; y = j.y0; r = v; }
    else if (v < j.n0 + j.n1) { W = j.W1; y = j.y1; r = v - j.n0; }
    else { W = j.W2; y = j.y2; r = v - j.n0 - j.n1; }
}
__device__ __forceinline__ float silu_times(float g, float u) { return g / (1.0f + expf(-g)) * u; }

/* v + the value 32 lanes away, and the sum of v over lanes n, n + 16, n + 32, n + 48 (in every one of them), by
 * gfx950's lane swaps: vector instructions, where a shuffle is a trip through LDS */
__device__ __forceinline__ float add_lane32(float v) {
    const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float sum_lane_groups(float v) {
    v = add_lane32(v);
    const auto q = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

/* wave64 sum: every lane ends up with the total */
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace qlin
#endif /* QLIN_DEVICE_H */
