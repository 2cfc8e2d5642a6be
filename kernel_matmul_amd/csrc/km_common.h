// Shared host/device definitions for the gfx950 KernelMatmul kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/kernel_matmul_amd.h"

#define KM_WAVE 64

namespace km {

typedef float float4v __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------
// Batch addressing.  The flat batch index (fastest dimension last) is split into its
// multi-index once per wavefront and turned into one element offset per tensor.  This is
// what native/common/accessor.cuh:5-102 of the reference does with compile-time ranks;
// here the rank is a run-time value so one binary serves every batch shape.
// ---------------------------------------------------------------------------------------
struct BatchShape {
    int rank;
    int sizes[KM_MAX_BATCH_RANK];
};

struct BatchStrides {
    long long s[KM_MAX_BATCH_RANK];
};

__device__ __forceinline__ void batch_multi_index(const BatchShape& shape, long long flat_index,
                                                  int (&idx)[KM_MAX_BATCH_RANK]) {
    // The number of batch items is below 2^31, so 32-bit division is enough.
    unsigned flat = (unsigned)flat_index;
#pragma unroll
    for (int d = KM_MAX_BATCH_RANK - 1; d >= 0; d--) {
        idx[d] = 0;
        if (d < shape.rank) {
            if (d == 0) {
                idx[0] = (int)flat;
            } else {
                const unsigned size = (unsigned)shape.sizes[d];
                const unsigned q = flat / size;
                idx[d] = (int)(flat - q * size);
                flat = q;
            }
        }
    }
}

__device__ __forceinline__ long long batch_offset(const BatchShape& shape,
                                                  const BatchStrides& strides,
                                                  const int (&idx)[KM_MAX_BATCH_RANK]) {
    long long off = 0;
#pragma unroll
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        if (d < shape.rank) {
            off += (long long)idx[d] * strides.s[d];
        }
    }
    return off;
}

// ---------------------------------------------------------------------------------------
// Workgroup -> work item mapping.  The hardware hands consecutive workgroup ids to the 8
// XCDs round-robin; each XCD has its own L2.  Items that touch neighbouring column windows
// of x2/rhs (consecutive row chunks, and all batch items of one row chunk) are therefore
// given to one XCD: xcd = id % 8 owns the contiguous item range [xcd*per_xcd, (xcd+1)*per_xcd).
// ---------------------------------------------------------------------------------------
#define KM_NUM_XCD 8

__device__ __forceinline__ long long xcd_item(unsigned block_id, long long per_xcd) {
    const unsigned xcd = block_id % KM_NUM_XCD;
    const unsigned slot = block_id / KM_NUM_XCD;
    return (long long)xcd * per_xcd + slot;
}

// ---------------------------------------------------------------------------------------
// Kernel functions.  The user-facing hyper-parameters are turned into the constants the
// inner loop wants once per wavefront (the reference does this with ~10 ATen launches per
// call, native/common/kernel_function.cuh:198-219).  All kernels are evaluated through the
// hardware base-2 exponential and the hardware sine/cosine that take their argument in
// revolutions, so cos(2*pi*f*d) is v_cos_f32(f*d):
//
//   rbf               sigma * exp(-d^2 / (2 l^2))                    = sgn * 2^(lsig - u^2)
//   spectral          sigma * exp(-d^2 / (2 l^2)) * cos(2 pi f d)    = sgn * 2^(lsig - u^2) * cos_rev(f d)
//   locally_periodic  sigma * exp(-d^2/(2 l^2) - (2/lp) sin^2(pi d / T))
//                                                  = sgn * 2^(lsig - u^2 - cl * sin_rev(d/(2T))^2)
//   with u = d * sqrt(log2(e)/2) / l, lsig = log2|sigma|, sgn = sign(sigma), cl = 2 log2(e) / lp.
//
// (reference formulas: native/common/kernel_function.cuh:25-58; gradients 92-163; chain
// rule back to the user parameters 221-251.)
// ---------------------------------------------------------------------------------------
#define KM_SQRT_HALF_LOG2E 0.84932180028801904272f /* sqrt(0.5 * log2(e)) */
#define KM_LOG2E 1.44269504088896340736f
#define KM_2LN2 1.38629436111989061883 /* 2 ln 2 */
#define KM_PI 3.14159265358979323846

struct KernelConsts {
    float s;     // u = d * s
    float f;     // phase (revolutions) = d * f
    float lsig;  // log2 |sigma|
    float cl;    // locally periodic: 2 log2(e) / lengthscale_periodic
    float sgn;   // sign of sigma (+1 / -1)
    float one;   // 1.0 that is only known at run time (keeps x * one + y an fma)
};

template <int KT>
struct KernelTraits;

template <>
struct KernelTraits<KM_KERNEL_RBF> {
    static constexpr int P = 2;
    static constexpr int SIGMA = 1;
};
template <>
struct KernelTraits<KM_KERNEL_SPECTRAL> {
    static constexpr int P = 3;
    static constexpr int SIGMA = 2;
};
template <>
struct KernelTraits<KM_KERNEL_LOCALLY_PERIODIC> {
    static constexpr int P = 4;
    static constexpr int SIGMA = 3;
};

template <int KT>
__device__ __forceinline__ KernelConsts make_consts(const float* __restrict__ params,
                                                    long long stride, bool fold_sigma) {
    KernelConsts c;
    const float l = params[0];
    c.s = KM_SQRT_HALF_LOG2E / fabsf(l);
    c.f = 0.0f;
    c.cl = 0.0f;
    if (KT == KM_KERNEL_SPECTRAL) {
        c.f = params[stride];
    }
    if (KT == KM_KERNEL_LOCALLY_PERIODIC) {
        c.cl = (2.0f * KM_LOG2E) / params[stride];
        c.f = 0.5f / params[2 * stride];
    }
    const float sigma = params[KernelTraits<KT>::SIGMA * stride];
    c.sgn = sigma < 0.0f ? -1.0f : 1.0f;
    c.lsig = fold_sigma ? log2f(fabsf(sigma)) : 0.0f;
    c.one = stride >= 0 ? 1.0f : 0.0f;  // strides are never negative
    return c;
}

// |K| without the sign of sigma (applied once per output element by the caller).
template <int KT>
__device__ __forceinline__ float kernel_value(float x1, float x2, const KernelConsts& c) {
    const float d = x1 - x2;
    const float u = d * c.s;
    const float arg = __builtin_fmaf(-u, u, c.lsig);
    if (KT == KM_KERNEL_RBF) {
        return __builtin_amdgcn_exp2f(arg);
    } else if (KT == KM_KERNEL_SPECTRAL) {
        const float e = __builtin_amdgcn_exp2f(arg);
        const float cs = __builtin_amdgcn_cosf(d * c.f);
        return e * cs;
    } else {
        const float sn = __builtin_amdgcn_sinf(d * c.f);
        const float w = sn * c.cl;
        return __builtin_amdgcn_exp2f(__builtin_fmaf(-w, sn, arg));
    }
}

// Sum over the 64 lanes of a wavefront (every lane receives the total).
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    return v;
}

// Accumulates the per-pair derivative terms.  acc[] meaning per kernel type:
//   rbf      : acc0 = sum C E u^2,  acc1 = sum C E
//   spectral : acc0 = sum C E cos u^2,  acc1 = sum C E sin d,  acc2 = sum C E cos
//   loc.per. : acc0 = sum C E u^2,  acc1 = sum C E sin^2,  acc2 = sum C E sin cos d,  acc3 = sum C E
// with E the kernel value without sigma.
template <int KT>
__device__ __forceinline__ void accumulate_pair(float x1, float x2, float coeff,
                                                const KernelConsts& kc, float (&acc)[KM_MAX_PARAMS]) {
    const float d = x1 - x2;
    const float u = d * kc.s;
    const float uu = u * u;
    if (KT == KM_KERNEL_RBF) {
        const float w = coeff * __builtin_amdgcn_exp2f(-uu);
        acc[0] = __builtin_fmaf(w, uu, acc[0]);
        acc[1] += w;
    } else if (KT == KM_KERNEL_SPECTRAL) {
        const float ph = d * kc.f;
        const float w = coeff * __builtin_amdgcn_exp2f(-uu);
        const float wc = w * __builtin_amdgcn_cosf(ph);
        const float ws = w * __builtin_amdgcn_sinf(ph);
        acc[0] = __builtin_fmaf(wc, uu, acc[0]);
        acc[1] = __builtin_fmaf(ws, d, acc[1]);
        acc[2] += wc;
    } else {
        const float ph = d * kc.f;
        const float sn = __builtin_amdgcn_sinf(ph);
        const float cs = __builtin_amdgcn_cosf(ph);
        const float q = sn * sn;
        const float w = coeff * __builtin_amdgcn_exp2f(__builtin_fmaf(-kc.cl, q, -uu));
        acc[0] = __builtin_fmaf(w, uu, acc[0]);
        acc[1] = __builtin_fmaf(w, q, acc[1]);
        acc[2] = __builtin_fmaf(w * (sn * cs), d, acc[2]);
        acc[3] += w;
    }
}

// Chain rule from the accumulated sums of accumulate_pair back to the user parameters
// (reference: native/common/kernel_function.cuh:221-251), written to g[0..P).
template <int KT>
__device__ __forceinline__ void finish_param_grad(double s0, double s1, double s2, double s3,
                                                  const float* __restrict__ params,
                                                  long long stride, float* __restrict__ g) {
    const double l = (double)params[0];
    const double sigma = (double)params[KernelTraits<KT>::SIGMA * stride];
    if (KT == KM_KERNEL_RBF) {
        g[0] = (float)(sigma * s0 * KM_2LN2 / l);
        g[1] = (float)s1;
    } else if (KT == KM_KERNEL_SPECTRAL) {
        g[0] = (float)(sigma * s0 * KM_2LN2 / l);
        g[1] = (float)(-2.0 * KM_PI * sigma * s1);
        g[2] = (float)s2;
    } else {
        const double lp = (double)params[stride];
        const double period = (double)params[2 * stride];
        g[0] = (float)(sigma * s0 * KM_2LN2 / l);
        g[1] = (float)(2.0 * sigma * s1 / (lp * lp));
        g[2] = (float)(4.0 * KM_PI * sigma * s2 / (lp * period * period));
        g[3] = (float)s3;
    }
}

}  // namespace km
