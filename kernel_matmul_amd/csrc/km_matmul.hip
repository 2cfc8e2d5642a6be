// Forward operator: out = K(x1, x2) @ rhs over per-row-block column ranges, K evaluated on
// the fly.  Two gfx950 implementations of the same contract:
//
//   fwd_mfma : each lane evaluates K entries directly in the A-operand layout of
//              v_mfma_f32_16x16x4_f32 and the K-tile x rhs-tile contraction runs on the
//              matrix pipe.  No LDS staging is needed: a wavefront owns whole rows, every
//              x2 / rhs element of its column range is loaded exactly once per wavefront
//              straight into the B-operand layout.
//   fwd_valu : one row per lane, the contraction is v_fma_f32 with wave-uniform x2 / rhs
//              operands fetched through the scalar (read-only) path.
//
// Computes what native/matmul/matmul.cu:13-157 of the reference computes.
#include "km_common.h"
#include "km_launch.h"

namespace km {

struct FwdArgs {
    BatchShape batch;
    long long num_batches;
    long long total_items;   // row chunks * batches
    long long items_per_xcd;
    int m, n, k;
    int chunks_per_block;    // 128 / rows per workgroup
    const float* x1;
    const float* x2;
    const float* rhs;
    const float* params;
    const int* start;
    const int* end;
    float* out;
    BatchStrides x1_bs, x2_bs, rhs_bs, params_bs, start_bs, end_bs;
    long long x1_s, x2_s, rhs_s0, rhs_s1, params_s, start_s, end_s;
};

// ---------------------------------------------------------------------------------------
// MFMA variant.
//
// v_mfma_f32_16x16x4_f32 operand layout (lane l of 64):
//   A[i][kk] (16x4)  : i = l % 16, kk = l / 16          -> K(x1[row i], x2[col kk])
//   B[kk][j] (4x16)  : kk = l / 16, j = l % 16          -> rhs[col kk][rhs column j]
//   D[i][j]  (16x16) : i = 4 * (l / 16) + v, j = l % 16 -> out[row i][rhs column j], v = 0..3
//
// A wavefront owns R groups of 16 rows and G groups of 16 rhs columns and walks its column
// range 4 columns per step: per step a lane loads one x2 value and G rhs values, evaluates
// R kernel entries and issues R*G MFMAs.  With S > 1 the S wavefronts of a workgroup split
// the column range and combine their accumulators through LDS in a fixed order.
// ---------------------------------------------------------------------------------------
template <int KT, int G, int R>
__global__ void __launch_bounds__(512) fwd_mfma(const FwdArgs a) {
    extern __shared__ float lds[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int S = blockDim.x >> 6;
    const int li = lane & 15;
    const int kk = lane >> 4;

    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (blockIdx.x / KM_NUM_XCD >= a.items_per_xcd || item >= a.total_items) {
        return;
    }
    const long long b = item % a.num_batches;
    const int chunk = (int)(item / a.num_batches);
    const int row_block = chunk / a.chunks_per_block;
    const int row0 = row_block * KM_BLOCK_SIZE + (chunk % a.chunks_per_block) * (16 * R);
    const int kbase = blockIdx.y * (16 * G);

    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
    const float* __restrict__ x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
    const float* __restrict__ rhs = a.rhs + batch_offset(a.batch, a.rhs_bs, bidx);
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    // Clamped to the valid columns: a symmetric pattern over fewer points than one block
    // reports end = block size > n (native/ranges/ranges.cpp:82-93 of the reference).
    const int range_start =
        max(a.start[batch_offset(a.batch, a.start_bs, bidx) + row_block * a.start_s], 0);
    const int range_end =
        min(a.end[batch_offset(a.batch, a.end_bs, bidx) + row_block * a.end_s], a.n);

    const KernelConsts kc = make_consts<KT>(params, a.params_s, true);

    // This wavefront's share of the column range, in whole steps of 4 columns.
    int col_begin = range_start;
    int col_end = range_end;
    if (S > 1) {
        const int width = range_end - range_start;
        const int per_wave = ((width + S - 1) / S + 3) & ~3;
        col_begin = range_start + wave * per_wave;
        col_end = min(range_end, col_begin + per_wave);
    }

    float x1v[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        const int row = min(row0 + 16 * r + li, a.m - 1);
        x1v[r] = x1[(long long)row * a.x1_s];
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
    const float* __restrict__ rhs_lane = rhs + (long long)(kbase + li) * a.rhs_s1;

    // Software pipeline: operands of step t+1 are requested before step t is evaluated.
    int col = col_begin + kk;
    float x2v = 0.0f;
    float bv[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        bv[g] = 0.0f;
    }
    if (col < col_end) {
        x2v = x2[(long long)col * a.x2_s];
#pragma unroll
        for (int g = 0; g < G; g++) {
            if (colmask[g]) {
                bv[g] = rhs_lane[(long long)col * a.rhs_s0 + (long long)(16 * g) * a.rhs_s1];
            }
        }
    }

    for (int c0 = col_begin; c0 < col_end; c0 += 4) {
        const int ncol = col + 4;
        float x2n = x2v;  // stays finite for masked-out lanes; their rhs operand is 0
        float bn[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            bn[g] = 0.0f;
        }
        if (ncol < col_end) {
            x2n = x2[(long long)ncol * a.x2_s];
#pragma unroll
            for (int g = 0; g < G; g++) {
                if (colmask[g]) {
                    bn[g] = rhs_lane[(long long)ncol * a.rhs_s0 + (long long)(16 * g) * a.rhs_s1];
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++) {
            const float kv = kernel_value<KT>(x1v[r], x2v, kc);
#pragma unroll
            for (int g = 0; g < G; g++) {
                acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv, bv[g], acc[r][g], 0, 0, 0);
            }
        }

        col = ncol;
        x2v = x2n;
#pragma unroll
        for (int g = 0; g < G; g++) {
            bv[g] = bn[g];
        }
    }

    float* __restrict__ out = a.out + b * (long long)a.m * a.k;

    if (S == 1) {
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int g = 0; g < G; g++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int row = row0 + 16 * r + 4 * kk + v;
                    if (row < a.m && colmask[g]) {
                        out[(long long)row * a.k + kbase + 16 * g + li] = acc[r][g][v] * kc.sgn;
                    }
                }
            }
        }
        return;
    }

    // Cross-wavefront reduction: lds[wave][slot][lane], slot = (r * G + g) * 4 + v.
    constexpr int SLOTS = R * G * 4;
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
        if (row < a.m && c < a.k) {
            out[(long long)row * a.k + c] = sum * kc.sgn;
        }
    }
}

// ---------------------------------------------------------------------------------------
// VALU variant: one workgroup of two wavefronts per 128-row block, one row per lane,
// KC rhs columns per pass.  x2[j] and rhs[j][0..KC) are the same for every lane, so they
// are read through uniform (scalar) loads and used as scalar operands of v_fma_f32.
// ---------------------------------------------------------------------------------------
template <int KT, int KC>
__global__ void __launch_bounds__(128) fwd_valu(const FwdArgs a) {
    const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
    if (blockIdx.x / KM_NUM_XCD >= a.items_per_xcd || item >= a.total_items) {
        return;
    }
    const long long b = item % a.num_batches;
    const int row_block = (int)(item / a.num_batches);
    const int row = row_block * KM_BLOCK_SIZE + threadIdx.x;
    const int kbase = blockIdx.y * KC;

    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
    const float* __restrict__ x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
    const float* __restrict__ rhs = a.rhs + batch_offset(a.batch, a.rhs_bs, bidx);
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    // Clamped to the valid columns: a symmetric pattern over fewer points than one block
    // reports end = block size > n (native/ranges/ranges.cpp:82-93 of the reference).
    const int range_start =
        max(a.start[batch_offset(a.batch, a.start_bs, bidx) + row_block * a.start_s], 0);
    const int range_end =
        min(a.end[batch_offset(a.batch, a.end_bs, bidx) + row_block * a.end_s], a.n);

    const KernelConsts kc = make_consts<KT>(params, a.params_s, true);
    const float x1v = x1[(long long)min(row, a.m - 1) * a.x1_s];

    float acc[KC];
#pragma unroll
    for (int c = 0; c < KC; c++) {
        acc[c] = 0.0f;
    }

    const int kc_valid = min(KC, a.k - kbase);
    const float* __restrict__ rhs_base = rhs + (long long)kbase * a.rhs_s1;
    if (kc_valid == KC) {
        for (int j = range_start; j < range_end; j++) {
            const float kv = kernel_value<KT>(x1v, x2[(long long)j * a.x2_s], kc);
            const float* __restrict__ rj = rhs_base + (long long)j * a.rhs_s0;
#pragma unroll
            for (int c = 0; c < KC; c++) {
                acc[c] = __builtin_fmaf(kv, rj[(long long)c * a.rhs_s1], acc[c]);
            }
        }
    } else {
        for (int j = range_start; j < range_end; j++) {
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
        float* __restrict__ out = a.out + (b * a.m + row) * (long long)a.k + kbase;
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
static hipError_t launch_mfma(const FwdArgs& a, int S, unsigned grid_x, unsigned grid_y,
                              hipStream_t stream) {
    const size_t lds = S > 1 ? (size_t)S * R * G * 4 * 64 * sizeof(float) : 0;
    hipLaunchKernelGGL((fwd_mfma<KT, G, R>), dim3(grid_x, grid_y, 1), dim3(64 * S, 1, 1), lds,
                       stream, a);
    return hipGetLastError();
}

template <int KT, int G>
static hipError_t launch_mfma_r(const FwdArgs& a, int R, int S, unsigned gx, unsigned gy,
                                hipStream_t stream) {
    switch (R) {
        case 8: return launch_mfma<KT, G, 8>(a, S, gx, gy, stream);
        case 4: return launch_mfma<KT, G, 4>(a, S, gx, gy, stream);
        case 2: return launch_mfma<KT, G, 2>(a, S, gx, gy, stream);
        default: return launch_mfma<KT, G, 1>(a, S, gx, gy, stream);
    }
}

template <int KT>
static hipError_t launch_mfma_g(const FwdArgs& a, int G, int R, int S, unsigned gx, unsigned gy,
                                hipStream_t stream) {
    switch (G) {
        case 4: return launch_mfma_r<KT, 4>(a, R, S, gx, gy, stream);
        case 2: return launch_mfma_r<KT, 2>(a, R, S, gx, gy, stream);
        default: return launch_mfma_r<KT, 1>(a, R, S, gx, gy, stream);
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

static void fill_strides(BatchStrides& dst, const int64_t* strides, int rank) {
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        dst.s[d] = d < rank ? strides[d] : 0;
    }
}

hipError_t launch_matmul(const MatmulProblem& p, const MatmulPlan& plan, hipStream_t stream) {
    FwdArgs a;
    a.batch.rank = p.batch_rank;
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        a.batch.sizes[d] = d < p.batch_rank ? (int)p.batch_sizes[d] : 1;
    }
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
    const int r = p.batch_rank;
    fill_strides(a.x1_bs, p.x1_strides, r);
    fill_strides(a.x2_bs, p.x2_strides, r);
    fill_strides(a.rhs_bs, p.rhs_strides, r);
    fill_strides(a.params_bs, p.params_strides, r);
    fill_strides(a.start_bs, p.start_strides, r);
    fill_strides(a.end_bs, p.end_strides, r);
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.rhs_s0 = p.rhs_strides[r];
    a.rhs_s1 = p.rhs_strides[r + 1];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];

    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    if (plan.variant == KM_VARIANT_VALU) {
        a.chunks_per_block = 1;
        a.total_items = row_blocks * p.num_batches;
    } else {
        a.chunks_per_block = KM_BLOCK_SIZE / (16 * plan.row_groups);
        a.total_items = row_blocks * a.chunks_per_block * p.num_batches;
    }
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    const unsigned grid_x = (unsigned)(a.items_per_xcd * KM_NUM_XCD);

    if (plan.variant == KM_VARIANT_VALU) {
        const unsigned grid_y = (unsigned)((p.k + plan.k_chunk - 1) / plan.k_chunk);
        switch (p.kernel_type) {
            case KM_KERNEL_RBF: return launch_valu<KM_KERNEL_RBF>(a, plan.k_chunk, grid_x, grid_y, stream);
            case KM_KERNEL_SPECTRAL: return launch_valu<KM_KERNEL_SPECTRAL>(a, plan.k_chunk, grid_x, grid_y, stream);
            default: return launch_valu<KM_KERNEL_LOCALLY_PERIODIC>(a, plan.k_chunk, grid_x, grid_y, stream);
        }
    }
    const int G = plan.k_chunk / 16;
    const unsigned grid_y = (unsigned)((p.k + plan.k_chunk - 1) / plan.k_chunk);
    switch (p.kernel_type) {
        case KM_KERNEL_RBF:
            return launch_mfma_g<KM_KERNEL_RBF>(a, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
        case KM_KERNEL_SPECTRAL:
            return launch_mfma_g<KM_KERNEL_SPECTRAL>(a, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
        default:
            return launch_mfma_g<KM_KERNEL_LOCALLY_PERIODIC>(a, G, plan.row_groups, plan.col_splits, grid_x, grid_y, stream);
    }
}

}  // namespace km
