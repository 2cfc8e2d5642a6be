// Forward operator: out = K(x1, x2) @ rhs over per-row-block column ranges, K evaluated on
// the fly (what native/matmul/matmul.cu:13-157 of the reference computes).  A wavefront owns
// whole rows and walks their column range; every x2 / rhs element of the range is loaded once
// per wavefront, coalesced, straight into MFMA operand layout.  gfx950 implementations of the
// same contract in this file:
//
//   fwd_table_f16 : split-fp16 contraction (below) with per-wavefront column tables in LDS
//                   (x2, scaled x2, and for spectral kernels cos / sin of the column phases:
//                   phase-split form).  rbf and spectral kernels, up to 16 rhs columns (the
//                   kernel the launch table picks for the headline shape); spectral kernels
//                   with 17 to 32 columns keep one accumulator set and take the cosine per
//                   entry from tabulated column phases.
//   fwd_mfma_f16  : K entries and rhs are each split into two fp16 terms (hi + lo, 22
//                   significant bits); the contraction is three v_mfma_f32_16x16x32_f16
//                   (hi*hi + hi*lo + lo*hi) accumulating in fp32, K evaluated directly per
//                   pair.  On gfx950 an MFMA keeps the SIMD's VALU (which evaluates K) from
//                   issuing for most of its duration, so matrix-pipe time adds to the VALU
//                   time: 3 x 17 clk per 16 x 32 tile here against 8 x 32 clk in fp32.
//   fwd_mfma_f32  : each lane evaluates K entries in the A-operand layout of
//                   v_mfma_f32_16x16x4_f32; the contraction is an fp32 MFMA.
//   fwd_valu      : one row per lane, contraction with v_fma_f32 on wave-uniform x2 / rhs
//                   operands fetched through the scalar (read-only) path.
//
// (fwd_block, which prepares the rhs operand once per workgroup of four row blocks, lives in
// km_matmul_block.hip.)  LDS carries the column tables of fwd_table_f16 and the fixed-order
// reduction when several wavefronts share a row range.
#include "km_batch.h"
#include "km_common.h"
#include "km_fwd.h"
#include "km_launch.h"

namespace km {

// Fixed-order reduction of the S wavefronts' accumulators through LDS and the masked store.
// lds[wave][slot][lane], slot = (r * G + g) * 4 + v in the MFMA D layout.
template <int G, int R>
__device__ __forceinline__ void reduce_and_store(const float4v (&acc)[R][G], float* lds, int S,
                                                 int wave, int lane, float* __restrict__ out,
                                                 int row0, int kbase, int m, int k) {
    constexpr int SLOTS = R * G * 4;
    const int li = lane & 15;
    const int kk = lane >> 4;
    float* mine = lds + (size_t)wave * SLOTS * 64;
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                mine[((r * G + g) * 4 + v) * 64 + lane] = acc[r][g][v];
            }
        }
    }
    __syncthreads();
    for (int slot = wave; slot < SLOTS; slot += S) {
        float sum = 0.0f;
        for (int w = 0; w < S; w++) {
            sum += lds[((size_t)w * SLOTS + slot) * 64 + lane];
        }
        const int v = slot & 3;
        const int g = (slot >> 2) % G;
        const int r = (slot >> 2) / G;
        const int row = row0 + 16 * r + 4 * kk + v;
        const int c = kbase + 16 * g + li;
        if (row < m && c < k) {
            out[(long long)row * k + c] = sum;
        }
    }
}

template <int G, int R>
__device__ __forceinline__ void store_direct(const float4v (&acc)[R][G], int lane,
                                             float* __restrict__ out, int row0, int kbase, int m,
                                             int k) {
    const int li = lane & 15;
    const int kk = lane >> 4;
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            const int c = kbase + 16 * g + li;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = row0 + 16 * r + 4 * kk + v;
                if (row < m && c < k) {
                    out[(long long)row * k + c] = acc[r][g][v];
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// fp32 MFMA variant.
//
// v_mfma_f32_16x16x4_f32 operand layout (lane l of 64):
//   A[i][kk] (16x4)  : i = l % 16, kk = l / 16          -> K(x1[row i], x2[col kk])
//   B[kk][j] (4x16)  : kk = l / 16, j = l % 16          -> rhs[col kk][rhs column j]
//   D[i][j]  (16x16) : i = 4 * (l / 16) + v, j = l % 16 -> out[row i][rhs column j], v = 0..3
//
// A wavefront owns R groups of 16 rows and G groups of 16 rhs columns and walks its column
// range 4 columns per step: per step a lane loads one x2 value and G rhs values, evaluates
// R kernel entries and issues R*G MFMAs.  With S > 1 the S wavefronts of a workgroup split
// the column range.
// ---------------------------------------------------------------------------------------
template <int KT, int G, int R>
__global__ void __launch_bounds__(512) fwd_mfma_f32(const FwdArgs a) {
    extern __shared__ float lds[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int S = blockDim.x >> 6;
    const int li = lane & 15;
    const int kk = lane >> 4;

    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    int chunk_in_block;
    const WaveView w = wave_view(a, item, a.chunks_per_block, &chunk_in_block);
    const int row0 = w.row_block * KM_BLOCK_SIZE + chunk_in_block * (16 * R);
    const int kbase = blockIdx.y * (16 * G);

    const KernelConsts kc = make_consts<KT>(w.params, a.params_s, true);

    // This wavefront's share of the column range, in whole steps of 4 columns.
    int col_begin = w.range_start;
    int col_end = w.range_end;
    if (S > 1) {
        const int width = max(w.range_end - w.range_start, 0);
        const int per_wave = ((width + S - 1) / S + 3) & ~3;
        col_begin = w.range_start + wave * per_wave;
        col_end = min(w.range_end, col_begin + per_wave);
    }

    float x1v[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = min(row0 + 16 * r + li, a.m - 1);
        x1v[r] = w.x1[(long long)row * a.x1_s];
    }

    float4v acc[R][G];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            acc[r][g] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    bool colmask[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        colmask[g] = kbase + 16 * g + li < a.k;
    }

    // Operand pointers advance by 4 columns per step.
    const float* x2p = w.x2 + (long long)(col_begin + kk) * a.x2_s;
    const float* rp = w.rhs + (long long)(col_begin + kk) * a.rhs_s0 + (long long)(kbase + li) * a.rhs_s1;
    const long long x2_step = 4 * a.x2_s;
    const long long r_step = 4 * a.rhs_s0;
    const long long g_step = 16 * a.rhs_s1;

    // Software pipeline: operands of step t+1 are requested before step t is evaluated.
    int col = col_begin + kk;
    float x2v = 0.0f;
    float bv[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        bv[g] = 0.0f;
    }
    if (col < col_end) {
        x2v = *x2p;
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (colmask[g]) {
                bv[g] = rp[g * g_step];
            }
        }
    }

    for (int c0 = col_begin; c0 < col_end; c0 += 4) {
        col += 4;
        x2p += x2_step;
        rp += r_step;
        float x2n = x2v;  // stays finite for masked-out lanes; their rhs operand is 0
        float bn[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            bn[g] = 0.0f;
        }
        if (col < col_end) {
            x2n = *x2p;
#pragma unroll
            for (int g = 0; g < G; g++) {
                if (colmask[g]) {
                    bn[g] = rp[g * g_step];
                }
            }
        }

        float kv[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            kv[r] = kernel_value<KT>(x1v[r], x2v, kc);
        }
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int g = 0; g < G; g++) {
                acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[r], bv[g], acc[r][g], 0, 0, 0);
            }
        }

        x2v = x2n;
#pragma unroll
        for (int g = 0; g < G; g++) {
            bv[g] = bn[g];
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            acc[r][g] *= kc.sgn;
        }
    }
    float* __restrict__ out = a.out + w.b * (long long)a.m * a.k;
    if (S == 1) {
        store_direct<G, R>(acc, lane, out, row0, kbase, a.m, a.k);
    } else {
        reduce_and_store<G, R>(acc, lds, S, wave, lane, out, row0, kbase, a.m, a.k);
    }
}

// ---------------------------------------------------------------------------------------
// Split-fp16 MFMA variant.
//
// v_mfma_f32_16x16x32_f16 operand layout (lane l of 64, 8 halves per operand register set):
//   A[i][8 kk + t] (16x32) : i = l % 16, kk = l / 16, t = 0..7 -> K(x1[row i], x2[col 8 kk + t])
//   B[8 kk + t][j] (32x16) : j = l % 16                         -> rhs[col 8 kk + t][rhs column j]
//   D as for the fp32 instruction.
//
// Every fp32 factor v is written as hi + lo with hi = fp16(v) and lo = fp16(v - hi)
// (round-to-nearest-even, v_cvt_pk_f16_f32), i.e. 22 significant bits, and the product is
// taken as hi*hi + hi*lo + lo*hi in the fp32 accumulator; the dropped lo*lo term is below
// 2^-22 relative.  To keep both factors inside the fp16 exponent range
//   - K is evaluated without sigma and scaled by 2^14 (folded into the exponent of the
//     base-2 exponential, so it costs nothing): |K| <= 2^14;
//   - each rhs column carries a running power-of-two scale per wavefront: when a step brings
//     a value that would exceed 2^15 after scaling, the scale is lowered and the column's
//     accumulators are multiplied by the (exact) ratio, so no pass over rhs is needed.
// Both scales and sigma are undone on the accumulators before they leave the wavefront.
// ---------------------------------------------------------------------------------------

// KS: log2 of the factor K / sigma is evaluated with (it keeps both halves inside the fp16 range).
template <int KT, int KS = KM_F16_KSCALE_LOG2>
__device__ __forceinline__ void kernel_pair_f16(float x1, float x2a, float x2b, const KernelConsts& c,
                                                float one, half2v* hi, half2v* lo) {
    // Two neighbouring columns at once so that the conversions pack.
    float2v kv;
    float ea[2], ca[2];
    const float x2s[2] = {x2a, x2b};
#pragma unroll
    for (int t = 0; t < 2; t++) {
        const float d = x1 - x2s[t];
        const float u = d * c.s;
        const float arg = __builtin_fmaf(-u, u, (float)KS);
        if (KT == KM_KERNEL_RBF) {
            ea[t] = __builtin_amdgcn_exp2f(arg);
            ca[t] = 1.0f;
        } else if (KT == KM_KERNEL_SPECTRAL) {
            ea[t] = __builtin_amdgcn_exp2f(arg);
            ca[t] = __builtin_amdgcn_cosf(d * c.f);
        } else {
            const float sn = __builtin_amdgcn_sinf(d * c.f);
            const float wv = sn * c.cl;
            ea[t] = __builtin_amdgcn_exp2f(__builtin_fmaf(-wv, sn, arg));
            ca[t] = 1.0f;
        }
        kv[t] = KT == KM_KERNEL_SPECTRAL ? ea[t] * ca[t] : ea[t];
    }
    const half2v h = __builtin_convertvector(kv, half2v);
    // Residuals of the exact products where there is one (`one` is a run-time 1.0 that keeps
    // the expression a fused multiply-add reading the fp16 operand directly).
    *hi = h;
    *lo = residual_f16x2(ea[0], KT == KM_KERNEL_SPECTRAL ? ca[0] : one, ea[1],
                         KT == KM_KERNEL_SPECTRAL ? ca[1] : one, h);
}

// Operands of one step of 32 columns for this lane: x2 and rhs at columns c0 + 8 kk + t.
// Full steps use a wave-uniform base (scalar registers) plus a loop-invariant 32-bit lane
// offset; the partial last step clamps the column to the range and zeroes the rhs operand of
// columns past it.
template <int G>
__device__ __forceinline__ void f16_load(const FwdArgs& a, const WaveView& w, int c0, int col_end,
                                         int kk, unsigned x2_lane, const unsigned (&rhs_lane)[G],
                                         float (&x2v)[8], float (&raw)[G][8]) {
    if (c0 + 32 <= col_end) {
        const float* x2u = w.x2 + (long long)c0 * a.x2_s;
        const float* ru = w.rhs + (long long)c0 * a.rhs_s0;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            x2v[t] = load_at(x2u + t * a.x2_s, x2_lane);
#pragma unroll
            for (int g = 0; g < G; g++) {
                raw[g][t] = load_at(ru + t * a.rhs_s0, rhs_lane[g]);
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int col = c0 + 8 * kk + t;
            const int colc = min(col, col_end - 1);
            x2v[t] = w.x2[(long long)colc * a.x2_s];
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float v = load_at(w.rhs + (long long)colc * a.rhs_s0, rhs_lane[g] - 4u * (unsigned)(8 * kk * a.rhs_s0));
                raw[g][t] = col < col_end ? v : 0.0f;
            }
        }
    }
}

// One step of 32 columns: convert this lane's 8 rhs values per column group to hi/lo halves
// (rescaling the accumulators first if a value would leave the fp16 range), then for every
// row group evaluate 8 kernel entries, split them and issue the three MFMAs.
// PARTS = 2 (phase-split form): every rhs value enters twice, multiplied by cb[] and by sb[]
// (|cb|, |sb| <= 1), into the accumulator groups g and G + g; both share the column's scale,
// which is taken from |rhs| alone.  PARTS = 1 with MULT: every rhs value is multiplied by cb[].
// SEP: x2v holds b = (x2 - ref) s and the entries are evaluated in the separable form (their
// column factors 2^(-b^2) come in through cb / sb).
// PAIRCOS (with SEP): the entries also carry the spectral kernel's cosine, taken per entry from
// the row phases pa[] and the column phases handed in through sb[] (revolutions).
template <int KT, int G, int R, int KS = KM_F16_KSCALE_LOG2, bool SEP = false, int PARTS = 1, bool MULT = false,
          bool PAIRCOS = false>
__device__ __forceinline__ void f16_step(const float (&x2v)[8], const float (&raw)[G][8],
                                         const float (&x1v)[R], const KernelConsts& kc,
                                         const bool (&colmask)[G], int (&shift)[G],
                                         float (&scale)[G], float4v (&acc)[R][G * PARTS], float ref = 0.0f,
                                         const float* cb = nullptr, const float* sb = nullptr,
                                         const float* pa = nullptr) {
    constexpr int GE = G * PARTS;
    half8v bhi[GE], blo[GE];
#pragma unroll
    for (int g = 0; g < G; g++) {
        // Largest magnitude of this rhs column over the step's 32 columns (the 4 lanes that
        // share the column hold 8 each).
        float m = 0.0f;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            m = fmaxf(m, fabsf(raw[g][t]));
        }
        m = column_max(m);
        const bool grow = colmask[g] && !(m * scale[g] < 32768.0f);
        if (__any(grow)) {
            if (grow) {
                // m < 2^e, so m * 2^(14 - e) < 2^14.
                const int e = __builtin_amdgcn_frexp_expf(m);
                const int new_shift = min(max(14 - e, -100), 100);
                const float factor = __builtin_ldexpf(1.0f, new_shift - shift[g]);
#pragma unroll
                for (int r = 0; r < R; r++) {
#pragma unroll
                    for (int part = 0; part < PARTS; part++) {
                        acc[r][part * G + g] *= factor;
                    }
                }
                shift[g] = new_shift;
                scale[g] = __builtin_ldexpf(1.0f, new_shift);
            }
        }
        float rv[8];
#pragma unroll
        for (int t = 0; t < 8; t++) {
            rv[t] = raw[g][t] * scale[g];
        }
        if (PARTS == 2) {
            float vc[8], vs[8];
#pragma unroll
            for (int t = 0; t < 8; t++) {
                vc[t] = rv[t] * cb[t];
                vs[t] = rv[t] * sb[t];
            }
            split_f16x8(vc, kc.one, &bhi[g], &blo[g]);
            split_f16x8(vs, kc.one, &bhi[G + g], &blo[G + g]);
        } else {
            if (MULT) {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    rv[t] *= cb[t];
                }
            }
            split_f16x8(rv, kc.one, &bhi[g], &blo[g]);
        }
    }

#pragma unroll
    for (int r = 0; r < R; r++) {
        half2v h2[4], l2[4];
        if (SEP) {
            // Row constants for this lane's 8 columns (ref: their reference point).
            const float av = (x1v[r] - ref) * kc.s;
            const float rb = __builtin_fmaf(-av, av, (float)KS);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                if (PAIRCOS) {
                    separable_pair_cos_f16(av, rb, x2v[2 * t], x2v[2 * t + 1], pa[r] - sb[2 * t],
                                           pa[r] - sb[2 * t + 1], &h2[t], &l2[t]);
                } else {
                    separable_pair_f16(av, rb, x2v[2 * t], x2v[2 * t + 1], kc.one, &h2[t], &l2[t]);
                }
            }
        } else {
#pragma unroll
            for (int t = 0; t < 4; t++) {
                kernel_pair_f16<KT, KS>(x1v[r], x2v[2 * t], x2v[2 * t + 1], kc, kc.one, &h2[t], &l2[t]);
            }
        }
        const half8v ahi = join_half2x4(h2);
        const half8v alo = join_half2x4(l2);
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bhi[g], acc[r][g], 0, 0, 0);
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, blo[g], acc[r][g], 0, 0, 0);
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bhi[g], acc[r][g], 0, 0, 0);
        }
        if (SEP) {
            // One row group at a time: the row constants of later groups are not formed ahead
            // of their use (registers); the MFMAs still overlap the next group's evaluation.
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// One step of 32 columns with the contraction in fp32 (v_mfma_f32_16x16x4_f32, 8 per row group and
// rhs column group): MFMA t of the step contracts the columns {8 kk + t}, so a lane evaluates its
// row against the same 8 consecutive columns as in the split-fp16 step and the column tables are
// shared.  Entries (K / sigma):
//   SEP      2^(a * 2b - a^2), the column factor 2^(-b^2) carried by cb / sb (spectral) or
//            multiplied into the rhs operand (rbf); x2v holds 2b
//   else     2^(-((x1 - x2) s)^2); x2v holds x2
//   spectral times cos(A_i - B_j) = cos A_i cos B_j + sin A_i sin B_j from the row's ca / sa and the
//            tabulated cb / sb: two full-rate operations instead of a phase product and a cosine.
template <int KT, int G, int R, bool SEP>
__device__ __forceinline__ void f32_step(const float (&x2v)[8], const float (&raw)[G][8],
                                         const float (&x1v)[R], const KernelConsts& kc,
                                         float4v (&acc)[R][G], float ref, const float (&cb)[8],
                                         const float (&sb)[8], const float (&ca)[R], const float (&sa)[R]) {
    float bv[G][8];
#pragma unroll
    for (int g = 0; g < G; g++) {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            bv[g][t] = (SEP && KT == KM_KERNEL_RBF) ? raw[g][t] * cb[t] : raw[g][t];
        }
    }
    // Two row groups at a time: their entries are evaluated first, then their MFMAs are issued
    // alternating between the two accumulators.
    constexpr int RI = R >= 2 ? 2 : 1;
#pragma unroll
    for (int r0 = 0; r0 < R; r0 += RI) {
        float kv[RI][8];
#pragma unroll
        for (int q = 0; q < RI; q++) {
            const int r = r0 + q;
            if (SEP) {
                const float av = (x1v[r] - ref) * kc.s;
                const float rb = -av * av;
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    kv[q][t] = __builtin_amdgcn_exp2f(__builtin_fmaf(av, x2v[t], rb));
                }
            } else {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const float u = (x1v[r] - x2v[t]) * kc.s;
                    kv[q][t] = __builtin_amdgcn_exp2f(-u * u);
                }
            }
            if (KT == KM_KERNEL_SPECTRAL) {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    kv[q][t] *= __builtin_fmaf(sa[r], sb[t], ca[r] * cb[t]);
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 8; t++) {
#pragma unroll
            for (int q = 0; q < RI; q++) {
#pragma unroll
                for (int g = 0; g < G; g++) {
                    acc[r0 + q][g] =
                        __builtin_amdgcn_mfma_f32_16x16x4f32(kv[q][t], bv[g][t], acc[r0 + q][g], 0, 0, 0);
                }
            }
        }
    }
}

// PF: request the next step's operands before evaluating the current one (costs 8 + 8 G
// registers; used for G = 1 where they are available).
template <int KT, int G, int R, bool PF>
__device__ __forceinline__ void fwd_mfma_f16_body(const FwdArgs& a, float* lds, const WaveView& wv,
                                                  int row0) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int S = blockDim.x >> 6;
    const int li = lane & 15;
    const int kk = lane >> 4;
    const int kbase = blockIdx.y * (16 * G);
    // The rhs column offset of this workgroup goes into the 64-bit base so that the 32-bit lane
    // offsets below span at most 24 rows and 16 G columns.
    WaveView w = wv;
    w.rhs += (long long)kbase * a.rhs_s1;

    const KernelConsts kc = make_consts<KT>(w.params, a.params_s, false);
    const float sigma = w.params[KernelTraits<KT>::SIGMA * a.params_s];

    // This wavefront's share of the column range, in whole steps of 32 columns.
    int col_begin = w.range_start;
    int col_end = w.range_end;
    if (S > 1) {
        const int width = max(w.range_end - w.range_start, 0);
        const int per_wave = ((width + S - 1) / S + 31) & ~31;
        col_begin = w.range_start + wave * per_wave;
        col_end = min(w.range_end, col_begin + per_wave);
    }

    float x1v[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = min(row0 + 16 * r + li, a.m - 1);
        x1v[r] = w.x1[(long long)row * a.x1_s];
    }

    // rhs columns past k read a valid column instead and are zeroed through their scale.
    bool colmask[G];
    unsigned rhs_lane[G];  // byte offset of (column 8 kk, rhs column of this lane)
    int shift[G];
    float scale[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int c = kbase + 16 * g + li;
        colmask[g] = c < a.k;
        rhs_lane[g] = 4u * (unsigned)(8 * kk * a.rhs_s0 + (min(c, a.k - 1) - kbase) * a.rhs_s1);
        // Start far up so that the first non-zero step sets the real scale.
        shift[g] = 100;
        scale[g] = colmask[g] ? __builtin_ldexpf(1.0f, 100) : 0.0f;
    }
    const unsigned x2_lane = 4u * (unsigned)(8 * kk * a.x2_s);

    float4v acc[R][G];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < G; g++) {
            acc[r][g] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    if (col_begin < col_end) {
        float x2v[8], raw[G][8];
        f16_load<G>(a, w, col_begin, col_end, kk, x2_lane, rhs_lane, x2v, raw);
        for (int c0 = col_begin; c0 < col_end; c0 += 32) {
            const bool more = c0 + 32 < col_end;
            if (PF) {
                float x2n[8], rawn[G][8];
                if (more) {
                    f16_load<G>(a, w, c0 + 32, col_end, kk, x2_lane, rhs_lane, x2n, rawn);
                }
                f16_step<KT, G, R>(x2v, raw, x1v, kc, colmask, shift, scale, acc);
                if (more) {
#pragma unroll
                    for (int t = 0; t < 8; t++) {
                        x2v[t] = x2n[t];
#pragma unroll
                        for (int g = 0; g < G; g++) {
                            raw[g][t] = rawn[g][t];
                        }
                    }
                }
            } else {
                f16_step<KT, G, R>(x2v, raw, x1v, kc, colmask, shift, scale, acc);
                if (more) {
                    f16_load<G>(a, w, c0 + 32, col_end, kk, x2_lane, rhs_lane, x2v, raw);
                }
            }
        }
    }

#pragma unroll
    for (int g = 0; g < G; g++) {
        const float unscale = __builtin_ldexpf(sigma, -shift[g] - KM_F16_KSCALE_LOG2);
#pragma unroll
        for (int r = 0; r < R; r++) {
            acc[r][g] *= unscale;
        }
    }
    float* __restrict__ out = a.out + w.b * (long long)a.m * a.k;
    if (S == 1) {
        store_direct<G, R>(acc, lane, out, row0, kbase, a.m, a.k);
    } else {
        reduce_and_store<G, R>(acc, lds, S, wave, lane, out, row0, kbase, a.m, a.k);
    }
}

template <int KT, int G, int R, bool PF>
__global__ void __launch_bounds__(512) fwd_mfma_f16(const FwdArgs a) {
    extern __shared__ float lds[];
    const ItemRef it = decode_item(a);
    if (!it.valid) {
        return;
    }
    int chunk_in_block;
    if constexpr (R == 8) {
        if (it.small) {
            const WaveView w = wave_view(a, it.item, 1, &chunk_in_block);
            fwd_mfma_f16_body<KT, G, 1, false>(a, lds, w, w.row_block * KM_BLOCK_SIZE + 16 * it.piece);
            return;
        }
    }
    const WaveView w = wave_view(a, it.item, a.chunks_per_block, &chunk_in_block);
    fwd_mfma_f16_body<KT, G, R, PF>(a, lds, w, w.row_block * KM_BLOCK_SIZE + chunk_in_block * (16 * R));
}

// ---------------------------------------------------------------------------------------
// Table kernel (rbf and spectral up to 16 rhs columns, spectral up to 32): split-fp16
// contraction with per-wavefront column tables in LDS.
//
// Phase-split form (spectral, one group of 16 rhs columns; with two groups the second
// accumulator set does not fit, and the entries carry cos(A_i - B_j) themselves, taken from
// the row's phase and the tabulated phase of the column).  With a reference point c per wavefront (its first row) and
// A_i = 2 pi f (x1_i - c), B_j = 2 pi f (x2_j - c):
//     cos(2 pi f (x1_i - x2_j)) = cos A_i cos B_j + sin A_i sin B_j
//     out[i,:] = cos A_i * sum_j E_ij (cos B_j rhs[j,:]) + sin A_i * sum_j E_ij (sin B_j rhs[j,:])
// with E_ij = exp(-d^2 / (2 l^2)) the Gaussian factor alone: the cosine leaves the per-pair
// work in exchange for twice the fp16 MFMAs.  cos B_j / sin B_j are needed once per column:
// each chunk of 512 columns is tabulated cooperatively by the wavefront (8 columns per lane)
// into LDS, and the steps read their 8 columns back as broadcast vector reads.  Phases are
// formed from an exact two-term difference to the reference point (once per row / column), so
// they are accurate to 3e-8 revolutions for any window width.
//
// Separable exponent.  A lane evaluates, per step, its row against 8 consecutive columns.
// With r the x2 value in the middle of these 8 columns, a = (x1_i - r) s and b_j = (x2_j - r) s:
//     2^(S - (a - b_j)^2) = 2^((S - a^2) + 2 a b_j) * 2^(-b_j^2)
// The last factor depends on the column alone and is tabulated with cos B_j / sin B_j (it
// multiplies the rhs operand); what is left per pair is ONE fma and one exp2, with the two row
// constants 2 a and S - a^2 formed once per row and 8 columns.  A chunk takes this form only
// when it loses nothing: every x2_j - r must be exact in fp32 (error-free transformation),
// every x1_i - r too (all coordinates involved have one sign and a spread below their smallest
// magnitude), and |b_j| <= 2, which bounds the evaluated factor by 2^(S + 4) -- inside the
// fp16 range for S = 11 -- and the column factor from below by 2^-4.  Otherwise (coordinates
// next to the origin, unsorted or widely spaced columns) the chunk evaluates
// 2^(S - ((x1_i - x2_j) s)^2) directly.
// ---------------------------------------------------------------------------------------
#define KM_PHASE_CHUNK 512
#define KM_PHASE_TABLE_FLOATS (4 * KM_PHASE_CHUNK + KM_PHASE_CHUNK / 8) /* per wavefront */

template <int G, bool BUFFER>
__device__ __forceinline__ void rhs_load(const FwdArgs& a, const WaveView& w, int c0, int col_end,
                                         int kk, const unsigned (&rhs_lane)[G], float (&raw)[G][8]) {
    if (c0 + 32 <= col_end) {
        if constexpr (BUFFER) {
            const buffer_rsrc ru = uniform_buffer(w.rhs + (long long)c0 * a.rhs_s0);
#pragma unroll
            for (int t = 0; t < 8; t++) {
#pragma unroll
                for (int g = 0; g < G; g++) {
                    raw[g][t] = buffer_at(ru, rhs_lane[g], 4u * (unsigned)(t * a.rhs_s0));
                }
            }
        } else {
            const float* ru = w.rhs + (long long)c0 * a.rhs_s0;
#pragma unroll
            for (int t = 0; t < 8; t++) {
#pragma unroll
                for (int g = 0; g < G; g++) {
                    raw[g][t] = load_at(ru + t * a.rhs_s0, rhs_lane[g]);
                }
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int col = c0 + 8 * kk + t;
            const int colc = min(col, col_end - 1);
#pragma unroll
            for (int g = 0; g < G; g++) {
                const float v = load_at(w.rhs + (long long)colc * a.rhs_s0, rhs_lane[g] - 4u * (unsigned)(8 * kk * a.rhs_s0));
                raw[g][t] = col < col_end ? v : 0.0f;
            }
        }
    }
}

// S wavefronts (this one is number `wave` of them) share the row range and split its columns;
// `slot` is the wavefront's table area in LDS.  With `overlay` the cross-wavefront reduction
// buffer lies over the table areas instead of behind them.
template <int KT, int G, int R, bool F32 = false>
__device__ __forceinline__ void fwd_table_body(const FwdArgs& a, float* lds, const WaveView& wv,
                                                   int row0, int S, int wave, int slot, bool overlay) {
    static_assert(KT == KM_KERNEL_SPECTRAL || KT == KM_KERNEL_RBF, "table kernel: rbf or spectral");
    // Spectral kernels: with one group of rhs columns the phase-split form (PHASE: the cosine
    // leaves the per-entry work for a second accumulator set); with two groups the doubled
    // accumulators do not fit, and the cosine is taken per entry from tabulated column phases
    // (PAIRCOS) - still the separable exponent and no phase arithmetic per entry.
    // F32: the contraction is an fp32 MFMA on the evaluated entries themselves (no split, no
    // scales); spectral entries take cos(A_i - B_j) from the tabulated cos B / sin B and the row's
    // cos A / sin A (TRIG).
    constexpr bool PHASE = !F32 && KT == KM_KERNEL_SPECTRAL && G == 1;
    constexpr bool PAIRCOS = !F32 && KT == KM_KERNEL_SPECTRAL && G > 1;
    constexpr bool TRIG = F32 && KT == KM_KERNEL_SPECTRAL;
    // Accumulator groups; phase-split: [cos part of g = 0..G), sin part of g = 0..G)].
    constexpr int GE = PHASE ? 2 * G : G;
    constexpr int CH = KM_PHASE_CHUNK;
    constexpr int PER_LANE = CH / 64;
    constexpr int KS = F32 ? 0 : KM_TABLE_KSCALE_LOG2;

    const int lane = threadIdx.x & 63;
    const int li = lane & 15;
    const int kk = lane >> 4;
    const int kbase = blockIdx.y * (16 * G);
    WaveView w = wv;  // rhs column offset of this workgroup in the 64-bit base, as above
    w.rhs += (long long)kbase * a.rhs_s1;

    const KernelConsts kc = make_consts<KT>(w.params, a.params_s, false);
    const float sigma = w.params[KernelTraits<KT>::SIGMA * a.params_s];
    const float c_ref = w.x1[(long long)min(row0, a.m - 1) * a.x1_s];

    int col_begin = w.range_start;
    int col_end = w.range_end;
    if (S > 1) {
        const int width = max(w.range_end - w.range_start, 0);
        const int per_wave = ((width + S - 1) / S + 31) & ~31;
        col_begin = w.range_start + wave * per_wave;
        col_end = min(w.range_end, col_begin + per_wave);
    }

    float x1v[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = min(row0 + 16 * r + li, a.m - 1);
        x1v[r] = w.x1[(long long)row * a.x1_s];
    }

    bool colmask[G];
    unsigned rhs_lane[G];
    int shift[G];
    float scale[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        const int c = kbase + 16 * g + li;
        rhs_lane[g] = 4u * (unsigned)(8 * kk * a.rhs_s0 + (min(c, a.k - 1) - kbase) * a.rhs_s1);
        colmask[g] = c < a.k;
        shift[g] = F32 ? 0 : 100;
        scale[g] = c < a.k ? __builtin_ldexpf(1.0f, 100) : 0.0f;
    }

    float4v acc[R][GE];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    // Per-wavefront table of the current chunk: x2, b = (x2 - r) s with r the x2 value in the
    // middle of each group of 8 columns, the two column factors of the rhs operand (cos B and
    // sin B, times 2^(-b^2) in the separable form; rbf: the first alone), and the r's.
    float* tab_x2 = lds + (size_t)slot * KM_PHASE_TABLE_FLOATS;
    float* tab_b = tab_x2 + CH;
    float* tab_cos = tab_b + CH;
    float* tab_sin = tab_cos + CH;
    float* tab_ref = tab_sin + CH;
    float* reduce_buffer = overlay ? lds : lds + (size_t)S * KM_PHASE_TABLE_FLOATS;

    float row_lo = __builtin_inff(), row_hi = -__builtin_inff();
    bool row_nan = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        row_lo = fminf(row_lo, x1v[r]);
        row_hi = fmaxf(row_hi, x1v[r]);
        row_nan = row_nan || x1v[r] != x1v[r];
    }
    wave_min_max(&row_lo, &row_hi);
    const bool rows_finite = !__any(row_nan);

    // Phases of this lane's rows against the reference point (per-entry cosine form only).
    float row_phase[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        row_phase[r] = PAIRCOS ? phase_rev(kc.f, x1v[r], c_ref) : 0.0f;
    }
    // Cosine and sine of the same phases (fp32 contraction: the lane's row of the A operand).
    float row_cos[R], row_sin[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const float th = TRIG ? phase_rev(kc.f, x1v[r], c_ref) : 0.0f;
        row_cos[r] = TRIG ? __builtin_amdgcn_cosf(th) : 1.0f;
        row_sin[r] = TRIG ? __builtin_amdgcn_sinf(th) : 0.0f;
    }

    // Tabulates the chunk [chunk0, chunk0 + 512) of this wavefront's columns; returns whether it
    // may take the separable form (then, if `allow`, the column factors already carry 2^(-b^2)).
    auto build = [&](int chunk0, bool allow) -> bool {
        const int chunk_end = min(chunk0 + CH, col_end);
        const int padded = (chunk_end - chunk0 + 31) & ~31;
        // Strides are below 2^22 elements, so 32 x 32 -> 64 bit products are enough.
        const float* x2c = w.x2 + (long long)chunk0 * a.x2_s;
        const unsigned x2_stride = (unsigned)a.x2_s;
        const int last = chunk_end - 1 - chunk0;
        // All loads of the chunk are requested before any is used: this lane's 8 columns
        // (lane, lane + 64, ...) and the reference point of column group `lane`; they go
        // straight to LDS, the arithmetic on them runs from there (few registers).
        {
            float xq[PER_LANE];
#pragma unroll
            for (int i = 0; i < PER_LANE; i++) {
                xq[i] = x2c[(unsigned long long)(unsigned)min(lane + 64 * i, last) * x2_stride];
            }
            const float ref_own = x2c[(unsigned long long)(unsigned)min(8 * lane + 4, last) * x2_stride];
#pragma unroll
            for (int i = 0; i < PER_LANE; i++) {
                tab_x2[lane + 64 * i] = xq[i];
            }
            tab_ref[lane] = ref_own;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        bool cols_ok = true;
        float lo = row_lo, hi = row_hi;
#pragma unroll 1
        for (int q = lane; q < padded; q += 64) {
            const float xv = tab_x2[q];
            const float ref = tab_ref[q >> 3];
            const float xd = xv - ref;
            const float bb = xd - xv;
            const float err = (xv - (xd - bb)) - (ref + bb);  // exact rounding error of xd
            const float b = xd * kc.s;
            tab_b[q] = b;
            if (PHASE || TRIG) {
                const float th = phase_rev(kc.f, xv, c_ref);
                tab_cos[q] = __builtin_amdgcn_cosf(th);
                tab_sin[q] = __builtin_amdgcn_sinf(th);
            } else {
                tab_cos[q] = 1.0f;
                if (PAIRCOS) {
                    tab_sin[q] = phase_rev(kc.f, xv, c_ref);  // the column's phase itself
                }
            }
            cols_ok = cols_ok && err == 0.0f && fabsf(b) <= KM_TABLE_SPAN;
            lo = fminf(lo, ref);
            hi = fmaxf(hi, ref);
        }
        wave_min_max(&lo, &hi);
        // x1 - r is exact for every row and reference point when all coordinates involved have
        // one sign and their spread does not exceed the smallest magnitude.
        const bool rows_ok = rows_finite && (lo > 0.0f || hi < 0.0f) && (hi - lo) <= fminf(fabsf(lo), fabsf(hi));
        const bool separable = allow && __all(cols_ok) && rows_ok;
        if (separable) {
            // The column factor 2^(-b^2) of the separable form joins the phase factors, and the
            // table keeps 2 b, the form the rows' exponent takes it in.
#pragma unroll 1
            for (int q = lane; q < padded; q += 64) {
                const float b = tab_b[q];
                const float wgt = __builtin_amdgcn_exp2f(-b * b);
                tab_b[q] = b + b;
                tab_cos[q] *= wgt;
                if (PHASE || TRIG) {
                    tab_sin[q] *= wgt;
                }
            }
        }
        // The table is written and read by this wavefront only.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        return separable;
    };

    // rhs operand of the current step.  The fp32 kernel (registers to spare) requests a chunk's
    // first step before the chunk is tabulated, so the two memory round trips overlap.
    float raw[G][8];
    auto request_first = [&](int chunk0) {
        if (F32) {
            rhs_load<G, !F32>(a, w, chunk0, min(chunk0 + CH, col_end), kk, rhs_lane, raw);
        }
    };

    // The steps of a tabulated chunk.
    auto steps = [&](int chunk0, auto sep_c) {
        constexpr bool SEP = decltype(sep_c)::value;
        const int chunk_end = min(chunk0 + CH, col_end);
        if (!F32) {
            rhs_load<G, !F32>(a, w, chunk0, chunk_end, kk, rhs_lane, raw);
        }
        for (int c0 = chunk0; c0 < chunk_end; c0 += 32) {
            const int off = c0 - chunk0 + 8 * kk;
            float x2v[8], cb[8], sb[8];
#pragma unroll
            for (int t = 0; t < 8; t += 4) {
                const float4v vx = *(const float4v*)((SEP ? tab_b : tab_x2) + off + t);
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    x2v[t + u] = vx[u];
                }
                if (PHASE || TRIG || SEP) {
                    const float4v vc = *(const float4v*)(tab_cos + off + t);
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        cb[t + u] = vc[u];
                    }
                }
                if (PHASE || TRIG || (PAIRCOS && SEP)) {
                    const float4v vs = *(const float4v*)(tab_sin + off + t);
#pragma unroll
                    for (int u = 0; u < 4; u++) {
                        sb[t + u] = vs[u];
                    }
                }
            }
            const float ref = SEP ? tab_ref[off >> 3] : 0.0f;
            // (chunks that cannot take the separable form evaluate the whole kernel directly)
            if constexpr (F32) {
                // The next step's rhs operand is requested before this step is evaluated.
                float rawn[G][8];
                if (c0 + 32 < chunk_end) {
                    rhs_load<G, !F32>(a, w, c0 + 32, chunk_end, kk, rhs_lane, rawn);
                }
                f32_step<KT, G, R, SEP>(x2v, raw, x1v, kc, acc, ref, cb, sb, row_cos, row_sin);
                if (c0 + 32 < chunk_end) {
#pragma unroll
                    for (int g = 0; g < G; g++) {
#pragma unroll
                        for (int t = 0; t < 8; t++) {
                            raw[g][t] = rawn[g][t];
                        }
                    }
                }
                continue;
            } else {
                f16_step<PAIRCOS ? KM_KERNEL_SPECTRAL : KM_KERNEL_RBF, G, R, KS, SEP, GE / G, SEP && !PHASE,
                         PAIRCOS && SEP>(x2v, raw, x1v, kc, colmask, shift, scale, acc, ref, cb, sb, row_phase);
            }
            if (c0 + 32 < chunk_end) {
                rhs_load<G, !F32>(a, w, c0 + 32, chunk_end, kk, rhs_lane, raw);
            }
        }
        // All reads of the table are done before the next chunk overwrites it.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    };

    // Separable chunks first; from the first chunk that cannot take that form on, the rest of
    // the range is evaluated directly (two loops in sequence rather than a choice inside one
    // loop: the register allocation of each stays on its own).
    int chunk0 = col_begin;
    bool tabulated = false;
    for (; chunk0 < col_end; chunk0 += CH) {
        tabulated = true;
        request_first(chunk0);
        if (!build(chunk0, true)) {
            break;
        }
        steps(chunk0, std::integral_constant<bool, true>{});
        tabulated = false;
    }
    for (; chunk0 < col_end; chunk0 += CH) {
        if (!tabulated) {
            request_first(chunk0);
            build(chunk0, false);
        }
        tabulated = false;
        steps(chunk0, std::integral_constant<bool, false>{});
    }

    // Power-of-two scales undone and sigma applied; phase-split:
    // out = sigma * (cos A * P + sin A * Q), with cos A / sin A formed once per row by the lane
    // that holds the row's coordinate (x1v: row 16 r + lane % 16) and fetched across lanes into
    // the accumulator layout (rows 16 r + 4 (lane / 16) + v).
    float4v res[R][G];
#pragma unroll
    for (int r = 0; r < R; r++) {
        float ca[4], sa[4];
        if (PHASE) {
            const float th = phase_rev(kc.f, x1v[r], c_ref);
            const float ca_own = __builtin_amdgcn_cosf(th);
            const float sa_own = __builtin_amdgcn_sinf(th);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                ca[v] = __shfl(ca_own, 4 * kk + v, 64);
                sa[v] = __shfl(sa_own, 4 * kk + v, 64);
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float up = __builtin_ldexpf(sigma, -shift[g] - KS);
#pragma unroll
            for (int v = 0; v < 4; v++) {
                if (PHASE) {
                    res[r][g][v] = ca[v] * (acc[r][g][v] * up) + sa[v] * (acc[r][GE - G + g][v] * up);
                } else {
                    res[r][g][v] = acc[r][g][v] * up;
                }
            }
        }
        // One row group at a time keeps the phase arithmetic of several groups from being
        // interleaved, which costs registers for nothing.
        __builtin_amdgcn_sched_barrier(0);
    }
    float* __restrict__ out = a.out + w.b * (long long)a.m * a.k;
    if (S == 1) {
        store_direct<G, R>(res, lane, out, row0, kbase, a.m, a.k);
    } else {
        if (overlay) {
            __syncthreads();  // every wavefront is done with its table
        }
        reduce_and_store<G, R>(res, reduce_buffer, S, wave, lane, out, row0, kbase, a.m, a.k);
    }
}

template <int KT, int G, int R, bool F32>
__device__ __forceinline__ void fwd_table_kernel(const FwdArgs& a, float* lds) {
    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    int chunk_in_block;
    const WaveView w = wave_view<true>(a, item, a.chunks_per_block, &chunk_in_block);
    // (the wavefront index is wave-uniform by construction; saying so keeps what is derived from
    // it in scalar registers)
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    fwd_table_body<KT, G, R, F32>(a, lds, w, w.row_block * KM_BLOCK_SIZE + chunk_in_block * (16 * R),
                                  blockDim.x >> 6, wave, wave, true);
}

template <int KT, int G, int R>
__global__ void __launch_bounds__(512, G == 1 ? 3 : 2) fwd_table_f16(const FwdArgs a) {
    extern __shared__ float lds[];
    fwd_table_kernel<KT, G, R, false>(a, lds);
}

// The same with the contraction as fp32 MFMAs (f32_step).
template <int KT, int G, int R>
__global__ void __launch_bounds__(512, G == 1 ? 3 : 2) fwd_table_f32(const FwdArgs a) {
    extern __shared__ float lds[];
    fwd_table_kernel<KT, G, R, true>(a, lds);
}

// Grouped launch of the table kernel for large problems (one wavefront per 128-row item, up to
// 16 rhs columns): workgroups of 4 wavefronts.  The first items of every XCD go one per
// wavefront, four to a workgroup; its last `tail_items` items are dispatched last, one per
// workgroup, with the four wavefronts splitting the item's column range (no repeated work) and
// adding their shares in a fixed order through LDS.  These quarter-length pieces fill the SIMDs
// while the last full items finish.
#define KM_GROUP_WAVES 4

template <int KT, bool F32>
__device__ __forceinline__ void fwd_table_grouped_kernel(const FwdArgs& a, float* lds) {
    // The wavefront index is wave-uniform by construction; saying so keeps the item and
    // everything derived from it (pointers, ranges, parameters) in scalar registers.
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned xcd = blockIdx.x % KM_NUM_XCD;
    const long long slot = blockIdx.x / KM_NUM_XCD;
    const long long main_items = a.items_per_xcd - a.tail_items;
    const long long main_groups = (main_items + KM_GROUP_WAVES - 1) / KM_GROUP_WAVES;
    const long long whole_tail = a.tail_items - a.tail_half_items;
    const bool split = slot >= main_groups;
    const bool halves = slot >= main_groups + whole_tail;
    long long local;
    int half = 0;
    if (!split) {
        local = slot * KM_GROUP_WAVES + wave;
        if (local >= main_items) {
            return;
        }
    } else if (!halves) {
        local = main_items + (slot - main_groups);
    } else {
        const long long u = slot - main_groups - whole_tail;
        local = main_items + whole_tail + u / 2;
        half = (int)(u % 2);
    }
    const long long item = (long long)xcd * a.items_per_xcd + local;
    if (item >= a.total_items) {
        return;  // uniform for the workgroup of a split item
    }
    int unused;
    const WaveView w = wave_view(a, item, 1, &unused);
    if (halves) {
        fwd_table_body<KT, 1, 4, F32>(a, lds, w, w.row_block * KM_BLOCK_SIZE + 64 * half, KM_GROUP_WAVES, wave, wave,
                                      true);
    } else {
        fwd_table_body<KT, 1, 8, F32>(a, lds, w, w.row_block * KM_BLOCK_SIZE, split ? KM_GROUP_WAVES : 1,
                                      split ? wave : 0, wave, true);
    }
}

template <int KT>
__global__ void __launch_bounds__(64 * KM_GROUP_WAVES, 3) fwd_table_f16_grouped(const FwdArgs a) {
    extern __shared__ float lds[];
    fwd_table_grouped_kernel<KT, false>(a, lds);
}

// The same launch shape for mid-size problems, where 128-row items would not fill the SIMDs
// once: the items are 64-row chunks, one per wavefront in workgroups of four; whatever exceeds
// whole rounds of one item per SIMD (the last `tail_items` of every XCD) is dispatched last, each
// split by columns over a workgroup.  A SIMD then runs one long wavefront and a few short ones
// beside it, where one wavefront per chunk would leave a fifth of the SIMDs with two and column
// shares for every chunk would put thousands of short-lived wavefronts through the dispatcher.
template <int KT>
__global__ void __launch_bounds__(64 * KM_GROUP_WAVES, 4) fwd_table_f16_grouped64(const FwdArgs a) {
    extern __shared__ float lds[];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const unsigned xcd = blockIdx.x % KM_NUM_XCD;
    const long long slot = blockIdx.x / KM_NUM_XCD;
    const long long main_items = a.items_per_xcd - a.tail_items;
    const long long main_groups = (main_items + KM_GROUP_WAVES - 1) / KM_GROUP_WAVES;
    const bool split = slot >= main_groups;
    long long local;
    if (!split) {
        local = slot * KM_GROUP_WAVES + wave;
        if (local >= main_items) {
            return;
        }
    } else {
        local = main_items + (slot - main_groups);
    }
    const long long item = (long long)xcd * a.items_per_xcd + local;
    if (item >= a.total_items) {
        return;  // uniform for the workgroup of a split item
    }
    int chunk_in_block;
    const WaveView w = wave_view<true>(a, item, 2, &chunk_in_block);
    fwd_table_body<KT, 1, 4, false>(a, lds, w, w.row_block * KM_BLOCK_SIZE + 64 * chunk_in_block,
                                    split ? KM_GROUP_WAVES : 1, split ? wave : 0, wave, true);
}

template <int KT>
__global__ void __launch_bounds__(64 * KM_GROUP_WAVES, 4) fwd_table_f32_grouped(const FwdArgs a) {
    extern __shared__ float lds[];
    fwd_table_grouped_kernel<KT, true>(a, lds);
}

// ---------------------------------------------------------------------------------------
// VALU variant: one workgroup of two wavefronts per 128-row block, one row per lane,
// KC rhs columns per pass.  x2[j] and rhs[j][0..KC) are the same for every lane, so they
// are read through uniform (scalar) loads and used as scalar operands of v_fma_f32.
// ---------------------------------------------------------------------------------------
template <int KT, int KC>
__global__ void __launch_bounds__(128) fwd_valu(const FwdArgs a) {
    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (item >= a.total_items) {
        return;
    }
    int unused;
    const WaveView w = wave_view(a, item, 1, &unused);
    const int row = w.row_block * KM_BLOCK_SIZE + threadIdx.x;
    const int kbase = blockIdx.y * KC;

    const KernelConsts kc = make_consts<KT>(w.params, a.params_s, true);
    const float x1v = w.x1[(long long)min(row, a.m - 1) * a.x1_s];

    float acc[KC];
#pragma unroll
    for (int c = 0; c < KC; c++) {
        acc[c] = 0.0f;
    }

    const int kc_valid = min(KC, a.k - kbase);
    const float* __restrict__ x2 = w.x2;
    const float* __restrict__ rhs_base = w.rhs + (long long)kbase * a.rhs_s1;
    if (kc_valid == KC) {
        for (int j = w.range_start; j < w.range_end; j++) {
            const float kv = kernel_value<KT>(x1v, x2[(long long)j * a.x2_s], kc);
            const float* __restrict__ rj = rhs_base + (long long)j * a.rhs_s0;
#pragma unroll
            for (int c = 0; c < KC; c++) {
                acc[c] = __builtin_fmaf(kv, rj[(long long)c * a.rhs_s1], acc[c]);
            }
        }
    } else {
        for (int j = w.range_start; j < w.range_end; j++) {
            const float kv = kernel_value<KT>(x1v, x2[(long long)j * a.x2_s], kc);
            const float* __restrict__ rj = rhs_base + (long long)j * a.rhs_s0;
#pragma unroll
            for (int c = 0; c < KC; c++) {
                const float rv = c < kc_valid ? rj[(long long)c * a.rhs_s1] : 0.0f;
                acc[c] = __builtin_fmaf(kv, rv, acc[c]);
            }
        }
    }

    if (row < a.m) {
        float* __restrict__ out = a.out + (w.b * a.m + row) * (long long)a.k + kbase;
#pragma unroll
        for (int c = 0; c < KC; c++) {
            if (c < kc_valid) {
                out[c] = acc[c] * kc.sgn;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Host dispatch.
// ---------------------------------------------------------------------------------------
template <int KT, int G, int R>
static hipError_t launch_mfma(const FwdArgs& a, int variant, int S, unsigned gx, unsigned gy,
                              hipStream_t stream) {
    const size_t lds = S > 1 ? (size_t)S * R * G * 4 * 64 * sizeof(float) : 0;
    constexpr bool HAS_TABLE_KERNEL = ((KT == KM_KERNEL_SPECTRAL || KT == KM_KERNEL_RBF) && G == 1) ||
                                      (KT == KM_KERNEL_SPECTRAL && G == 2);
    if (variant == KM_VARIANT_MFMA_F16) {
        // The table kernel exists for the shapes the launch table can pick (register budget).
        if constexpr (HAS_TABLE_KERNEL) {
            // The cross-wavefront reduction buffer lies over the tables (every wavefront is done
            // with its table by then): less LDS per workgroup, more workgroups per CU.
            const size_t table = (size_t)S * KM_PHASE_TABLE_FLOATS * sizeof(float);
            hipLaunchKernelGGL((fwd_table_f16<KT, G, R>), dim3(gx, gy, 1), dim3(64 * S, 1, 1),
                               table > lds ? table : lds, stream, a);
        } else {
            return hipErrorInvalidConfiguration;
        }
    } else if (variant == KM_VARIANT_MFMA_F16_DIRECT) {
        // Wide rhs tiles with many row groups exceed the register file; the launch table never
        // picks them.
        if constexpr (G * R <= 16) {
            hipLaunchKernelGGL((fwd_mfma_f16<KT, G, R, G == 1>), dim3(gx, gy, 1), dim3(64 * S, 1, 1), lds, stream, a);
        } else {
            return hipErrorInvalidConfiguration;
        }
    } else if (variant == KM_VARIANT_MFMA_F32) {
        if constexpr ((KT == KM_KERNEL_SPECTRAL || KT == KM_KERNEL_RBF) && G <= 2) {
            const size_t table = (size_t)S * KM_PHASE_TABLE_FLOATS * sizeof(float);
            hipLaunchKernelGGL((fwd_table_f32<KT, G, R>), dim3(gx, gy, 1), dim3(64 * S, 1, 1),
                               table > lds ? table : lds, stream, a);
        } else {
            return hipErrorInvalidConfiguration;
        }
    } else {
        hipLaunchKernelGGL((fwd_mfma_f32<KT, G, R>), dim3(gx, gy, 1), dim3(64 * S, 1, 1), lds, stream, a);
    }
    return hipGetLastError();
}

template <int KT, int G>
static hipError_t launch_mfma_r(const FwdArgs& a, int variant, int R, int S, unsigned gx,
                                unsigned gy, hipStream_t stream) {
    switch (R) {
        case 8: return launch_mfma<KT, G, 8>(a, variant, S, gx, gy, stream);
        case 4: return launch_mfma<KT, G, 4>(a, variant, S, gx, gy, stream);
        case 2: return launch_mfma<KT, G, 2>(a, variant, S, gx, gy, stream);
        default: return launch_mfma<KT, G, 1>(a, variant, S, gx, gy, stream);
    }
}

template <int KT>
static hipError_t launch_mfma_g(const FwdArgs& a, int variant, int G, int R, int S, unsigned gx,
                                unsigned gy, hipStream_t stream) {
    switch (G) {
        case 4: return launch_mfma_r<KT, 4>(a, variant, R, S, gx, gy, stream);
        case 2: return launch_mfma_r<KT, 2>(a, variant, R, S, gx, gy, stream);
        default: return launch_mfma_r<KT, 1>(a, variant, R, S, gx, gy, stream);
    }
}

template <int KT>
static hipError_t launch_valu(const FwdArgs& a, int KC, unsigned gx, unsigned gy,
                              hipStream_t stream) {
    if (KC == 16) {
        hipLaunchKernelGGL((fwd_valu<KT, 16>), dim3(gx, gy, 1), dim3(128, 1, 1), 0, stream, a);
    } else if (KC == 8) {
        hipLaunchKernelGGL((fwd_valu<KT, 8>), dim3(gx, gy, 1), dim3(128, 1, 1), 0, stream, a);
    } else {
        hipLaunchKernelGGL((fwd_valu<KT, 4>), dim3(gx, gy, 1), dim3(128, 1, 1), 0, stream, a);
    }
    return hipGetLastError();
}

void fill_fwd_args(const MatmulProblem& p, FwdArgs* args) {
    FwdArgs& a = *args;
    const int r = p.batch_rank;
    const int64_t* const strides[6] = {p.x1_strides, p.x2_strides, p.rhs_strides,
                                       p.params_strides, p.start_strides, p.end_strides};
    BatchStrides* outs[6] = {&a.x1_bs, &a.x2_bs, &a.rhs_bs, &a.params_bs, &a.start_bs, &a.end_bs};
    collapse_batch<6>(r, p.batch_sizes, strides, &a.batch, outs);
    a.num_batches = p.num_batches;
    a.m = (int)p.m;
    a.n = (int)p.n;
    a.k = (int)p.k;
    a.x1 = p.x1;
    a.x2 = p.x2;
    a.rhs = p.rhs;
    a.params = p.params;
    a.start = p.start;
    a.end = p.end;
    a.out = p.out;
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.rhs_s0 = p.rhs_strides[r];
    a.rhs_s1 = p.rhs_strides[r + 1];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];
    a.total_items = 0;
    a.items_per_xcd = 0;
    a.chunks_per_block = 1;
    a.tail_items = 0;
    a.tail_half_items = 0;
}

hipError_t launch_matmul(const MatmulProblem& p, const MatmulPlan& plan, hipStream_t stream) {
    if (plan.variant == KM_VARIANT_BLOCK) {
        return launch_matmul_block(p, plan, stream);
    }
    FwdArgs a;
    fill_fwd_args(p, &a);

    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    if (plan.variant == KM_VARIANT_VALU) {
        a.chunks_per_block = 1;
        a.total_items = row_blocks * p.num_batches;
    } else {
        a.chunks_per_block = KM_BLOCK_SIZE / (16 * plan.row_groups);
        a.total_items = row_blocks * a.chunks_per_block * p.num_batches;
    }
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    a.tail_items = 0;
    a.tail_half_items = 0;
    unsigned grid_x = (unsigned)(a.items_per_xcd * KM_NUM_XCD);
    const unsigned grid_y = (unsigned)((p.k + plan.k_chunk - 1) / plan.k_chunk);
    // Tail balancing (direct split-fp16 kernel, one wavefront per 128-row block): whatever does
    // not fill all 128 SIMDs of an XCD evenly is cut into 16-row pieces and dispatched last.
    if (plan.variant == KM_VARIANT_MFMA_F16_DIRECT && plan.row_groups == 8 && plan.col_splits == 1 &&
        plan.tail_balance && a.items_per_xcd >= 2 * 128) {
        a.tail_items = (int)(a.items_per_xcd % 128);
        grid_x = (unsigned)((a.items_per_xcd - a.tail_items + 8LL * a.tail_items) * KM_NUM_XCD);
    }

    if (plan.variant == KM_VARIANT_VALU) {
        switch (p.kernel_type) {
            case KM_KERNEL_RBF: return launch_valu<KM_KERNEL_RBF>(a, plan.k_chunk, grid_x, grid_y, stream);
            case KM_KERNEL_SPECTRAL: return launch_valu<KM_KERNEL_SPECTRAL>(a, plan.k_chunk, grid_x, grid_y, stream);
            default: return launch_valu<KM_KERNEL_LOCALLY_PERIODIC>(a, plan.k_chunk, grid_x, grid_y, stream);
        }
    }
    if (plan.variant == KM_VARIANT_MFMA_F16 && plan.group_tail >= 0 && plan.row_groups == 4 && plan.col_splits == 1 &&
        plan.k_chunk == 16 && p.kernel_type != KM_KERNEL_LOCALLY_PERIODIC) {
        // 64-row items (a.total_items / a.items_per_xcd already count them)
        a.tail_items = (int)(plan.group_tail < a.items_per_xcd ? plan.group_tail : a.items_per_xcd);
        a.tail_half_items = 0;
        const long long main_groups = (a.items_per_xcd - a.tail_items + KM_GROUP_WAVES - 1) / KM_GROUP_WAVES;
        const unsigned gx = (unsigned)((main_groups + a.tail_items) * KM_NUM_XCD);
        const size_t table = (size_t)KM_GROUP_WAVES * KM_PHASE_TABLE_FLOATS * sizeof(float);
        if (p.kernel_type == KM_KERNEL_SPECTRAL) {
            hipLaunchKernelGGL((fwd_table_f16_grouped64<KM_KERNEL_SPECTRAL>), dim3(gx, grid_y, 1),
                               dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
        } else {
            hipLaunchKernelGGL((fwd_table_f16_grouped64<KM_KERNEL_RBF>), dim3(gx, grid_y, 1),
                               dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
        }
        return hipGetLastError();
    }
    if ((plan.variant == KM_VARIANT_MFMA_F16 || plan.variant == KM_VARIANT_MFMA_F32) && plan.group_tail >= 0 &&
        plan.row_groups == 8 && plan.col_splits == 1 && plan.k_chunk == 16 &&
        p.kernel_type != KM_KERNEL_LOCALLY_PERIODIC) {
        a.tail_items = (int)(plan.group_tail < a.items_per_xcd ? plan.group_tail : a.items_per_xcd);
        a.tail_half_items = (int)(plan.group_tail_halves < a.tail_items ? plan.group_tail_halves : a.tail_items);
        const long long main_groups = (a.items_per_xcd - a.tail_items + KM_GROUP_WAVES - 1) / KM_GROUP_WAVES;
        const unsigned gx = (unsigned)((main_groups + a.tail_items + a.tail_half_items) * KM_NUM_XCD);
        const size_t table = (size_t)KM_GROUP_WAVES * KM_PHASE_TABLE_FLOATS * sizeof(float);
        static_assert(KM_GROUP_WAVES * 8 * 4 * 64 <= KM_GROUP_WAVES * KM_PHASE_TABLE_FLOATS,
                      "the reduction buffer of a split item must fit over the tables");
        if (plan.variant == KM_VARIANT_MFMA_F32) {
            if (p.kernel_type == KM_KERNEL_SPECTRAL) {
                hipLaunchKernelGGL((fwd_table_f32_grouped<KM_KERNEL_SPECTRAL>), dim3(gx, grid_y, 1),
                                   dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
            } else {
                hipLaunchKernelGGL((fwd_table_f32_grouped<KM_KERNEL_RBF>), dim3(gx, grid_y, 1),
                                   dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
            }
        } else if (p.kernel_type == KM_KERNEL_SPECTRAL) {
            hipLaunchKernelGGL((fwd_table_f16_grouped<KM_KERNEL_SPECTRAL>), dim3(gx, grid_y, 1),
                               dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
        } else {
            hipLaunchKernelGGL((fwd_table_f16_grouped<KM_KERNEL_RBF>), dim3(gx, grid_y, 1),
                               dim3(64 * KM_GROUP_WAVES, 1, 1), table, stream, a);
        }
        return hipGetLastError();
    }
    const int G = plan.k_chunk / 16;
    switch (p.kernel_type) {
        case KM_KERNEL_RBF:
            return launch_mfma_g<KM_KERNEL_RBF>(a, plan.variant, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
        case KM_KERNEL_SPECTRAL:
            return launch_mfma_g<KM_KERNEL_SPECTRAL>(a, plan.variant, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
        default:
            return launch_mfma_g<KM_KERNEL_LOCALLY_PERIODIC>(a, plan.variant, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
    }
}

}  // namespace km
