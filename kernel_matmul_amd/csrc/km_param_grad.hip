// Hyper-parameter gradient of sum_{(i,j) in mask} C[i,j] K[i,j] with C = left @ right^T.
// Serves the reference operators matmul_bwd (left = out_grad, right = rhs;
// native/matmul_bwd/matmul_bwd.cu:12-221) and bilinear_derivative
// (native/bilinear_derivative/bilinear_derivative.cu:12-183), which compute the same sum.
//
// Pass 1 has two forms.  Feature form (param_grad_features, rbf and spectral kernels with
// narrow vectors; described at the kernel): the sums are polynomials in the rows' coordinate
// times contractions of the Gaussian factor with a handful of column features, computed like
// the forward table kernel.  Pairwise form (param_grad_partial, every kernel; also the
// per-item fallback of the feature form): a wavefront owns 128 rows and a share of the row
// block's column range.  Per 16-column chunk and 16-row group the coefficient tile C (16x16) is
// formed on the matrix pipe from left/right (v_mfma_f32_16x16x4_f32 over the vector
// columns); its D layout gives each lane 4 (row, col) pairs, for which the lane evaluates
// the kernel derivatives and accumulates per-lane sums.  The sums are combined across the
// wavefront with DPP/permute shuffles and written as one partial row per wavefront.
// Pass 2 (param_grad_reduce): one workgroup per batch item adds the partial rows in a
// fixed order in fp64 and applies the chain rule back to the user parameters
// (native/common/kernel_function.cuh:221-251).  No atomics: results are reproducible.
#include <cstdio>

#include "km_batch.h"
#include "km_common.h"
#include "km_fwd.h"
#include "km_launch.h"

namespace km {

// The first 240 bytes are everything a wavefront of the pairwise kernel reads when the batch
// shape has collapsed to at most one dimension: contiguous, so that its prologue fetches the
// argument block with a few wide scalar loads issued together instead of a chain of dependent
// ones.
struct GradArgs {
    long long num_batches;
    long long total_items;  // row blocks * col splits * batches
    long long items_per_xcd;
    long long partial_rows;  // total_items / num_batches
    int m, n, c;
    int col_splits;
    const float* x1;
    const float* x2;
    const float* left;
    const float* right;
    const float* params;
    const int* start;
    const int* end;
    float* partials;  // [num_batches][row_blocks * col_splits][KM_MAX_PARAMS]
    long long first_bs[7];  // stride of the first batch dimension of x1, x2, left, right, params, start, end
    long long x1_s, x2_s, left_s0, left_s1, right_s0, right_s1, params_s, start_s, end_s;
    BatchShape batch;
    BatchStrides x1_bs, x2_bs, left_bs, right_bs, params_bs, start_bs, end_bs;
};

// One item of the pairwise form: R groups of 16 rows from row0 against the columns
// [col_begin, col_end), sums written to `prow` (KM_MAX_PARAMS floats).
// TL > 0: the vector width c is at most 4*TL and the left operand stays in registers.
// TL == 0: any c; the left operand is re-read (from L1/L2) for every column chunk.
//
// FAST: every inner stride is non-negative and at most KM_GRAD_FAST_STRIDE elements (the host
// checks).  Addresses are then a wave-uniform 64-bit base, advanced on the scalar unit, plus a
// loop-invariant 32-bit lane offset formed once with 24-bit multiplies; the general form pays
// a 64-bit vector multiplication (four quarter-rate instructions) per load, which for a short
// column share is a third of the wavefront's issue time (48 row operands against three chunks).
#define KM_GRAD_FAST_STRIDE (1 << 21)

template <int KT, int TL, int R, bool FAST = false>
__device__ __forceinline__ void pairwise_item(const GradArgs& a, const float* __restrict__ x1,
                                              const float* __restrict__ x2, const float* __restrict__ left,
                                              const float* __restrict__ right, const KernelConsts& kc,
                                              int row0, int col_begin, int col_end,
                                              float* __restrict__ prow) {
    const int lane = threadIdx.x & 63;
    const int li = lane & 15;
    const int kk = lane >> 4;

    // x1 for the 4 rows per row group this lane owns in the D layout, and the left operand
    // (A layout): row = row0 + 16 r + li, vector column = 4 t + kk.
    constexpr int TLR = TL > 0 ? TL : 1;
    float x1q[R][4];
    float lreg[R][TLR];
    // FAST: lane offsets (bytes) of the vector columns 4 t + kk, clamped into the row, and whether
    // the column exists.
    unsigned left_col[TLR], right_col[TLR];
    bool col_used[TLR];
    if (FAST) {
        const unsigned x1_s = (unsigned)a.x1_s, l0 = (unsigned)a.left_s0, l1 = (unsigned)a.left_s1;
        const unsigned r1 = (unsigned)a.right_s1;
#pragma unroll
        for (int t = 0; t < TLR; t++) {
            const unsigned cc = (unsigned)min(4 * t + kk, a.c - 1);
            col_used[t] = 4 * t + kk < a.c;
            left_col[t] = 4u * __umul24(cc, l1);
            right_col[t] = 4u * __umul24(cc, r1);
        }
        // (buffer loads: base and row offset in scalar registers, see uniform_buffer)
        const buffer_rsrc x1_rows = uniform_buffer(x1 + (long long)row0 * a.x1_s);
        const buffer_rsrc left_rows = uniform_buffer(left + (long long)row0 * a.left_s0);
        if (row0 + 16 * R <= a.m) {
            const unsigned x1_lane = 4u * __umul24(4u * (unsigned)kk, x1_s);
            const unsigned left_lane = 4u * __umul24((unsigned)li, l0);
            unsigned left_lane_col[TLR];
#pragma unroll
            for (int t = 0; t < TLR; t++) {
                left_lane_col[t] = left_lane + left_col[t];
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    x1q[r][v] = buffer_at(x1_rows, x1_lane, 4u * (unsigned)(16 * r + v) * x1_s);
                }
                if (TL > 0) {
#pragma unroll
                    for (int t = 0; t < TLR; t++) {
                        const float value = buffer_at(left_rows, left_lane_col[t], 4u * (unsigned)(16 * r) * l0);
                        lreg[r][t] = col_used[t] ? value : 0.0f;
                    }
                }
            }
        } else {
            // The last row block: rows past m read row m - 1 (x1) or count as zero (left).
            const int last = a.m - 1 - row0;
#pragma unroll
            for (int r = 0; r < R; r++) {
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const unsigned rel = (unsigned)min(16 * r + 4 * kk + v, last);
                    x1q[r][v] = buffer_at(x1_rows, 4u * __umul24(rel, x1_s), 0u);
                }
                if (TL > 0) {
                    const int rel = 16 * r + li;
                    const unsigned row_off = 4u * __umul24((unsigned)min(rel, last), l0);
#pragma unroll
                    for (int t = 0; t < TLR; t++) {
                        const float value = buffer_at(left_rows, row_off + left_col[t], 0u);
                        lreg[r][t] = (rel <= last && col_used[t]) ? value : 0.0f;
                    }
                }
            }
        }
    } else {
#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int row = min(row0 + 16 * r + 4 * kk + v, a.m - 1);
                x1q[r][v] = x1[(long long)row * a.x1_s];
            }
        }
        if (TL > 0) {
#pragma unroll
            for (int r = 0; r < R; r++) {
                const int row = row0 + 16 * r + li;
#pragma unroll
                for (int t = 0; t < TLR; t++) {
                    const int cc = 4 * t + kk;
                    lreg[r][t] = (row < a.m && cc < a.c)
                                     ? left[(long long)row * a.left_s0 + (long long)cc * a.left_s1]
                                     : 0.0f;
                }
            }
        }
    }

    float acc[KM_MAX_PARAMS] = {0.0f, 0.0f, 0.0f, 0.0f};

    // Operands of a chunk of 16 columns: x2 of column n0 + li and, with the left operand in
    // registers, the right operand's values (column n0 + li, vector column 4 t + kk), zero outside
    // the range.  They are requested one chunk ahead.
    const unsigned x2_lane = FAST ? 4u * __umul24((unsigned)li, (unsigned)a.x2_s) : 0u;
    unsigned right_lane_col[TLR];
#pragma unroll
    for (int t = 0; t < TLR; t++) {
        right_lane_col[t] = FAST ? 4u * __umul24((unsigned)li, (unsigned)a.right_s0) + right_col[t] : 0u;
    }
    auto load_chunk = [&](int n0, float* x2v, float (&rv)[TLR]) {
        const int col = n0 + li;
        const int col_c = min(col, col_end - 1);
        if (FAST) {
            const buffer_rsrc x2_cols = uniform_buffer(x2 + (long long)n0 * a.x2_s);
            const buffer_rsrc right_cols = uniform_buffer(right + (long long)n0 * a.right_s0);
            // (values of columns past the range or the vector width are zeroed where they are
            // used, one chunk later: a select here would wait for the load at once)
            if (n0 + 16 <= col_end) {
                *x2v = buffer_at(x2_cols, x2_lane, 0u);
                if (TL > 0) {
#pragma unroll
                    for (int t = 0; t < TLR; t++) {
                        rv[t] = buffer_at(right_cols, right_lane_col[t], 0u);
                    }
                }
            } else {
                const unsigned rel = (unsigned)(col_c - n0);
                *x2v = buffer_at(x2_cols, 4u * __umul24(rel, (unsigned)a.x2_s), 0u);
                if (TL > 0) {
                    const unsigned col_off = 4u * __umul24(rel, (unsigned)a.right_s0);
#pragma unroll
                    for (int t = 0; t < TLR; t++) {
                        rv[t] = buffer_at(right_cols, col_off + right_col[t], 0u);
                    }
                }
            }
            return;
        }
        *x2v = x2[(long long)col_c * a.x2_s];
        if (TL > 0) {
#pragma unroll
            for (int t = 0; t < TLR; t++) {
                const int cc = 4 * t + kk;
                rv[t] = (col < col_end && cc < a.c)
                            ? right[(long long)col_c * a.right_s0 + (long long)cc * a.right_s1]
                            : 0.0f;
            }
        }
    };
    float x2_next = 0.0f, rv_next[TLR];
    if (col_begin < col_end) {
        load_chunk(col_begin, &x2_next, rv_next);
    }

    for (int n0 = col_begin; n0 < col_end; n0 += 16) {
        const int col = n0 + li;
        const bool col_ok = col < col_end;
        const int col_c = min(col, col_end - 1);
        const float x2v = x2_next;
        float rvs[TLR];
#pragma unroll
        for (int t = 0; t < TLR; t++) {
            rvs[t] = (!FAST || (col_ok && col_used[t])) ? rv_next[t] : 0.0f;
        }
        if (n0 + 16 < col_end) {
            load_chunk(n0 + 16, &x2_next, rv_next);
        }

        float4v coef[R];
#pragma unroll
        for (int r = 0; r < R; r++) {
            coef[r] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }

        if (TL > 0) {
#pragma unroll
            for (int t = 0; t < TLR; t++) {
#pragma unroll
                for (int r = 0; r < R; r++) {
                    coef[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(lreg[r][t], rvs[t], coef[r], 0, 0, 0);
                }
            }
        } else {
            for (int c0 = 0; c0 < a.c; c0 += 4) {
                const int cc = c0 + kk;
                const float rv = (col_ok && cc < a.c)
                                     ? right[(long long)col_c * a.right_s0 + (long long)cc * a.right_s1]
                                     : 0.0f;
#pragma unroll
                for (int r = 0; r < R; r++) {
                    const int row = row0 + 16 * r + li;
                    const float lv = (row < a.m && cc < a.c)
                                         ? left[(long long)row * a.left_s0 + (long long)cc * a.left_s1]
                                         : 0.0f;
                    coef[r] = __builtin_amdgcn_mfma_f32_16x16x4f32(lv, rv, coef[r], 0, 0, 0);
                }
            }
        }

#pragma unroll
        for (int r = 0; r < R; r++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                accumulate_pair<KT>(x1q[r][v], x2v, coef[r][v], kc, acc);
            }
        }
    }

#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        const float total = wave_sum(acc[p]);
        if (lane == 0) {
            prow[p] = total;
        }
    }
}

// Per-wavefront decode shared by the two kernels: item -> (batch item, row chunk, column
// split), the batch item's pointers, and the wavefront's share of the row block's range.
struct GradItem {
    long long b, rest;
    int row0, col_begin, col_end;
    int width;  // columns of the row block's whole range (all shares)
    const float* x1;
    const float* x2;
    const float* left;
    const float* right;
    const float* params;
};

// FAST: all counts are below 2^31 (the host checks): 32-bit divisions.
template <bool FAST = false>
__device__ __forceinline__ bool grad_item(const GradArgs& a, int rows_per_item, int col_step, GradItem* g) {
    int split, chunk;
    if (FAST) {
        const unsigned item = (blockIdx.x % KM_NUM_XCD) * (unsigned)a.items_per_xcd + blockIdx.x / KM_NUM_XCD;
        if (item >= (unsigned)a.total_items) {
            return false;
        }
        const unsigned batches = (unsigned)a.num_batches;
        const unsigned rest = item / batches;
        g->b = item - rest * batches;
        g->rest = rest;
        chunk = (int)(rest / (unsigned)a.col_splits);
        split = (int)(rest - (unsigned)chunk * (unsigned)a.col_splits);
    } else {
        const long long item = xcd_item(blockIdx.x, a.items_per_xcd);
        if (item >= a.total_items) {
            return false;
        }
        g->b = item % a.num_batches;
        g->rest = item / a.num_batches;
        split = (int)(g->rest % a.col_splits);
        chunk = (int)(g->rest / a.col_splits);
    }
    const int chunks_per_block = KM_BLOCK_SIZE / rows_per_item;
    const int row_block = chunk / chunks_per_block;
    g->row0 = row_block * KM_BLOCK_SIZE + (chunk % chunks_per_block) * rows_per_item;

    long long off_start, off_end;
    if (FAST) {
        // (launched for collapsed batch shapes only)
        g->x1 = a.x1 + g->b * a.first_bs[0];
        g->x2 = a.x2 + g->b * a.first_bs[1];
        g->left = a.left + g->b * a.first_bs[2];
        g->right = a.right + g->b * a.first_bs[3];
        g->params = a.params + g->b * a.first_bs[4];
        off_start = g->b * a.first_bs[5];
        off_end = g->b * a.first_bs[6];
    } else if (a.batch.rank <= 1) {
        // The usual case after the host has collapsed the batch dimensions: one stride per tensor.
        g->x1 = a.x1 + g->b * a.x1_bs.s[0];
        g->x2 = a.x2 + g->b * a.x2_bs.s[0];
        g->left = a.left + g->b * a.left_bs.s[0];
        g->right = a.right + g->b * a.right_bs.s[0];
        g->params = a.params + g->b * a.params_bs.s[0];
        off_start = g->b * a.start_bs.s[0];
        off_end = g->b * a.end_bs.s[0];
    } else {
        int bidx[KM_MAX_BATCH_RANK];
        batch_multi_index(a.batch, g->b, bidx);
        g->x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
        g->x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
        g->left = a.left + batch_offset(a.batch, a.left_bs, bidx);
        g->right = a.right + batch_offset(a.batch, a.right_bs, bidx);
        g->params = a.params + batch_offset(a.batch, a.params_bs, bidx);
        off_start = batch_offset(a.batch, a.start_bs, bidx);
        off_end = batch_offset(a.batch, a.end_bs, bidx);
    }
    int range_start = a.start[off_start + row_block * a.start_s];
    int range_end = a.end[off_end + row_block * a.end_s];
    range_start = max(range_start, 0);
    range_end = min(range_end, a.n);
    // Column share of this wavefront, in whole steps of col_step columns.
    const int width = max(range_end - range_start, 0);
    g->width = width;
    const int per_split = ((width + a.col_splits - 1) / a.col_splits + col_step - 1) & ~(col_step - 1);
    g->col_begin = range_start + split * per_split;
    g->col_end = min(range_end, g->col_begin + per_split);
    return true;
}

template <int KT, int TL, bool FAST>
__global__ void __launch_bounds__(64) param_grad_partial(const GradArgs a) {
    if (FAST) {
        // All of the argument block's hot part is requested here, in one go: left to the
        // compiler the loads are issued where each value is first used, one round trip to the
        // scalar cache after the other (six before the first row operand is requested).
        asm volatile("" ::"s"(a.num_batches), "s"(a.total_items), "s"(a.items_per_xcd), "s"(a.partial_rows),
                     "s"(a.m), "s"(a.n), "s"(a.c), "s"(a.col_splits), "s"(a.x1), "s"(a.x2), "s"(a.left),
                     "s"(a.right), "s"(a.params), "s"(a.start), "s"(a.end), "s"(a.partials));
        asm volatile("" ::"s"(a.first_bs[0]), "s"(a.first_bs[1]), "s"(a.first_bs[2]), "s"(a.first_bs[3]),
                     "s"(a.first_bs[4]), "s"(a.first_bs[5]), "s"(a.first_bs[6]), "s"(a.x1_s), "s"(a.x2_s),
                     "s"(a.left_s0), "s"(a.left_s1), "s"(a.right_s0), "s"(a.right_s1), "s"(a.params_s),
                     "s"(a.start_s), "s"(a.end_s));
    }
    GradItem g;
    if (!grad_item<FAST>(a, KM_BLOCK_SIZE, 16, &g)) {
        return;
    }
    const KernelConsts kc = make_consts<KT>(g.params, a.params_s, false);
    pairwise_item<KT, TL, 8, FAST>(a, g.x1, g.x2, g.left, g.right, kc, g.row0, g.col_begin, g.col_end,
                                   a.partials + (g.b * a.partial_rows + g.rest) * KM_MAX_PARAMS);
}

// ---------------------------------------------------------------------------------------
// Feature form of pass 1 (rbf and spectral kernels, narrow vector widths).
//
// With a reference point c0 per wavefront (the middle row of its rows), h_i = (x1_i - c0) s,
// g_j = (x2_j - c0) s, A_i / B_j the phases of x1_i - c0 / x2_j - c0 and E_ij the Gaussian
// factor,  u_ij = h_i - g_j,  cos(A_i - B_j) = cA cB + sA sB,  sin(A_i - B_j) = sA cB - cA sB,
// every sum the gradient needs is a polynomial in h_i times a row-wise contraction of E with
// column features F_j = {cB, sB, cB g, sB g, cB g^2, sB g^2} (rbf: {1, g, g^2}):
//     M[i, c, f] = sum_j E_ij right[j, c] F_jf              T_f[i] = sum_c left[i, c] M[i, c, f]
//     sum C E cos      = sum_i  cA T0 + sA T1
//     sum C E cos u^2  = sum_i  cA (h^2 T0 - 2 h T2 + T4) + sA (h^2 T1 - 2 h T3 + T5)
//     sum C E sin d    = sum_i  [sA (h T0 - T2) - cA (h T1 - T3)] / s
// M is exactly what the forward table kernel computes for an rhs of (number of features) x c
// columns: one fma + one exp2 per pair (separable exponent), the hi/lo split, and the
// split-fp16 MFMAs; the per-pair cosine, sine and the products of the pairwise form are gone.
// The polynomial in h cancels leading terms of size h^2 against a result of size u^2 ~ 1, so the
// form is only used while |h_i| <= 12 (measured on 1e5 points: the 22-bit products then leave
// up to 2e-5 of the gradient's largest component, 1e-6 for |h| <= 6), |g_j| <= 48 (dynamic range
// of the fp16 operands), every chunk of columns admits the separable exponent and the row block's
// range has at least 64 columns (with a handful of columns nothing averages the rounding of the
// row sums, measured up to 7e-5 of sum |terms| for a single column against 4e-6 from 64 columns
// on, and the pairwise form costs next to nothing there); an item that fails any of these is
// redone in the pairwise form.
// ---------------------------------------------------------------------------------------
#define KM_GF_CHUNK 512
#define KM_GF_MAX_FEATURES 6
#define KM_GF_MAX_WIDTH 10 /* widest vector the feature form takes */
/* column tables of a chunk (b, features, reference points) or, in the epilogue, the row weights */
#define KM_GF_HEAD_FLOATS ((1 + KM_GF_MAX_FEATURES) * KM_GF_CHUNK + KM_GF_CHUNK / 8)
#define KM_GF_TABLE_FLOATS (KM_GF_HEAD_FLOATS + KM_BLOCK_SIZE * KM_GF_MAX_WIDTH)
#define KM_GF_HMAX 12.0f
#define KM_GF_GMAX 48.0f
#define KM_GF_MIN_WIDTH 64 /* columns in the row block's range */

template <int KT, int GE, int R, int TL>
__global__ void __launch_bounds__(64, 2) param_grad_features(const GradArgs a) {
    static_assert(KT == KM_KERNEL_RBF || KT == KM_KERNEL_SPECTRAL, "feature form: rbf or spectral");
    static_assert(R == 8, "128 rows per item (row weights: two rows per lane)");
    static_assert(KM_BLOCK_SIZE * KM_GF_MAX_FEATURES * 3 <= KM_GF_HEAD_FLOATS,
                  "the row weights must fit in front of the staged rows of left");
    constexpr bool PHASE = KT == KM_KERNEL_SPECTRAL;
    constexpr int NF = PHASE ? 6 : 3;
    constexpr int CH = KM_GF_CHUNK;
    constexpr int KS = KM_TABLE_KSCALE_LOG2;
    extern __shared__ float lds[];
    float* tab_b = lds;                    // 2 (x2 - r) s per column, r: reference of its 8 columns
    float* tab_f = lds + CH;               // [NF][CH] column features times 2^(-b^2)
    float* tab_ref = lds + (1 + KM_GF_MAX_FEATURES) * CH;
    // (the epilogue's row weights, [16 R][NF][3], later overlay everything up to here)
    float* tab_left = lds + KM_GF_HEAD_FLOATS;  // [16 R][c]: this item's rows of `left` (epilogue)

    GradItem g;
    if (!grad_item(a, 16 * R, 32, &g)) {
        return;
    }
    const int lane = threadIdx.x;
    const int li = lane & 15;
    const int kk = lane >> 4;
    const KernelConsts kc = make_consts<KT>(g.params, a.params_s, false);
    float* __restrict__ prow = a.partials + (g.b * a.partial_rows + g.rest) * KM_MAX_PARAMS;
    const int row0 = g.row0;
    const int col_begin = g.col_begin, col_end = g.col_end;

    // Operand column t = 16 ge + li of group ge holds (feature f, vector column c) = (t / c, t % c).
    int feat[GE], vcol[GE];
    bool used[GE];
    unsigned right_lane[GE];
#pragma unroll
    for (int ge = 0; ge < GE; ge++) {
        const int t = 16 * ge + li;
        used[ge] = t < NF * a.c;
        feat[ge] = used[ge] ? t / a.c : 0;
        vcol[ge] = used[ge] ? t % a.c : 0;
        right_lane[ge] = (unsigned)(8 * kk * a.right_s0 + vcol[ge] * a.right_s1);
    }

    float x1v[R];
#pragma unroll
    for (int r = 0; r < R; r++) {
        x1v[r] = g.x1[(long long)min(row0 + 16 * r + li, a.m - 1) * a.x1_s];
    }
    const float c0 = g.x1[(long long)min(row0 + 8 * R, a.m - 1) * a.x1_s];

    // This item's rows of `left` go to LDS now (coalesced, overlapping the first table) and are
    // read back in the epilogue; rows past m are zero.
    for (int e = lane; e < 16 * R * a.c; e += 64) {
        const int lr = e / a.c, lc = e - lr * a.c;
        tab_left[e] = row0 + lr < a.m
                          ? g.left[(long long)(row0 + lr) * a.left_s0 + (long long)lc * a.left_s1]
                          : 0.0f;
    }

    float row_lo = __builtin_inff(), row_hi = -__builtin_inff();
    bool row_nan = false;
#pragma unroll
    for (int r = 0; r < R; r++) {
        row_lo = fminf(row_lo, x1v[r]);
        row_hi = fmaxf(row_hi, x1v[r]);
        row_nan = row_nan || x1v[r] != x1v[r];
    }
    wave_min_max(&row_lo, &row_hi);
    bool ok = !__any(row_nan) && fmaxf(fabsf(row_hi - c0), fabsf(row_lo - c0)) * kc.s <= KM_GF_HMAX &&
              g.width >= KM_GF_MIN_WIDTH;

    int shift[GE];
    float scale[GE];
#pragma unroll
    for (int ge = 0; ge < GE; ge++) {
        shift[ge] = 100;
        scale[ge] = used[ge] ? __builtin_ldexpf(1.0f, 100) : 0.0f;
    }
    float4v acc[R][GE];
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int ge = 0; ge < GE; ge++) {
            acc[r][ge] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    for (int chunk0 = col_begin; ok && chunk0 < col_end; chunk0 += CH) {
        const int chunk_end = min(chunk0 + CH, col_end);
        const int padded = (chunk_end - chunk0 + 31) & ~31;
        const float* x2c = g.x2 + (long long)chunk0 * a.x2_s;
        const unsigned x2_stride = (unsigned)a.x2_s;
        const int last = chunk_end - 1 - chunk0;
        // All loads of the chunk first (4 columns per lane and the reference point of column
        // group `lane`), staged through the feature area of the table.
        {
            float xq[CH / 64];
#pragma unroll
            for (int i = 0; i < CH / 64; i++) {
                xq[i] = x2c[(unsigned long long)(unsigned)min(lane + 64 * i, last) * x2_stride];
            }
            const float ref_own = x2c[(unsigned long long)(unsigned)min(8 * (lane & (CH / 8 - 1)) + 4, last) * x2_stride];
#pragma unroll
            for (int i = 0; i < CH / 64; i++) {
                tab_b[lane + 64 * i] = xq[i];
            }
            if (lane < CH / 8) {
                tab_ref[lane] = ref_own;
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        bool cols_ok = true;
        float lo = row_lo, hi = row_hi;
#pragma unroll 1
        for (int q = lane; q < padded; q += 64) {
            const float xv = tab_b[q];
            const float ref = tab_ref[q >> 3];
            const float xd = xv - ref;
            const float bb = xd - xv;
            const float err = (xv - (xd - bb)) - (ref + bb);  // exact rounding error of xd
            const float b = xd * kc.s;
            const float gq = (xv - c0) * kc.s;
            const float wgt = __builtin_amdgcn_exp2f(-b * b);
            float p0 = wgt, p1 = 0.0f;
            if (PHASE) {
                const float th = phase_rev(kc.f, xv, c0);
                p0 = wgt * __builtin_amdgcn_cosf(th);
                p1 = wgt * __builtin_amdgcn_sinf(th);
            }
            tab_b[q] = b + b;  // the form the rows' exponent takes it in
            if (PHASE) {
                tab_f[0 * CH + q] = p0;
                tab_f[1 * CH + q] = p1;
                tab_f[2 * CH + q] = p0 * gq;
                tab_f[3 * CH + q] = p1 * gq;
                tab_f[4 * CH + q] = p0 * gq * gq;
                tab_f[5 * CH + q] = p1 * gq * gq;
            } else {
                tab_f[0 * CH + q] = p0;
                tab_f[1 * CH + q] = p0 * gq;
                tab_f[2 * CH + q] = p0 * gq * gq;
            }
            cols_ok = cols_ok && err == 0.0f && fabsf(b) <= KM_TABLE_SPAN && fabsf(gq) <= KM_GF_GMAX;
            lo = fminf(lo, ref);
            hi = fmaxf(hi, ref);
        }
        wave_min_max(&lo, &hi);
        // x1 - r is exact for every row and reference point when all coordinates involved have
        // one sign and their spread does not exceed the smallest magnitude.
        const bool rows_ok = (lo > 0.0f || hi < 0.0f) && (hi - lo) <= fminf(fabsf(lo), fabsf(hi));
        ok = __all(cols_ok) && rows_ok;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (!ok) {
            break;
        }

        // Steps of 32 columns.  The operands of a step are requested at its start (no prefetch:
        // the registers go to the accumulators; other wavefronts cover the latency).
        float raw[GE][8];
        auto load = [&](int c0s) {
            if (c0s + 32 <= chunk_end) {
                const float* ru = g.right + (long long)c0s * a.right_s0;
#pragma unroll
                for (int t = 0; t < 8; t++) {
#pragma unroll
                    for (int ge = 0; ge < GE; ge++) {
                        raw[ge][t] = (ru + t * a.right_s0)[right_lane[ge]];
                    }
                }
            } else {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const int col = c0s + 8 * kk + t;
                    const int colc = min(col, chunk_end - 1);
#pragma unroll
                    for (int ge = 0; ge < GE; ge++) {
                        const float v = g.right[(long long)colc * a.right_s0 + vcol[ge] * a.right_s1];
                        raw[ge][t] = col < chunk_end ? v : 0.0f;
                    }
                }
            }
        };
        load(chunk0);
        for (int c0s = chunk0; c0s < chunk_end; c0s += 32) {
            const int off = c0s - chunk0 + 8 * kk;
            float bv[8];
            {
                const float4v v0 = *(const float4v*)(tab_b + off);
                const float4v v1 = *(const float4v*)(tab_b + off + 4);
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    bv[u] = v0[u];
                    bv[4 + u] = v1[u];
                }
            }
            const float ref = tab_ref[off >> 3];
            half8v bhi[GE], blo[GE];
#pragma unroll
            for (int ge = 0; ge < GE; ge++) {
                const float* fp = tab_f + feat[ge] * CH + off;
                const float4v m0 = *(const float4v*)fp;
                const float4v m1 = *(const float4v*)(fp + 4);
                // Largest magnitude of this operand column over the step (the 4 lanes that share
                // it hold 8 columns each), features included (they are not bounded by one).
                float rv[8];
                float m = 0.0f;
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    rv[t] = raw[ge][t] * (t < 4 ? m0[t & 3] : m1[t & 3]);
                    m = fmaxf(m, fabsf(rv[t]));
                }
                m = column_max(m);
                const bool grow = used[ge] && !(m * scale[ge] < 32768.0f);
                if (__any(grow)) {
                    if (grow) {
                        // m < 2^e, so m * 2^(14 - e) < 2^14.
                        const int e = __builtin_amdgcn_frexp_expf(m);
                        const int new_shift = min(max(14 - e, -100), 100);
                        const float factor = __builtin_ldexpf(1.0f, new_shift - shift[ge]);
#pragma unroll
                        for (int r = 0; r < R; r++) {
                            acc[r][ge] *= factor;
                        }
                        shift[ge] = new_shift;
                        scale[ge] = __builtin_ldexpf(1.0f, new_shift);
                    }
                }
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    rv[t] *= scale[ge];
                }
                split_f16x8(rv, kc.one, &bhi[ge], &blo[ge]);
            }
            if (c0s + 32 < chunk_end) {
                load(c0s + 32);
            }
#pragma unroll
            for (int r = 0; r < R; r++) {
                half2v h2[4], l2[4];
                const float av = (x1v[r] - ref) * kc.s;
                const float rb = __builtin_fmaf(-av, av, (float)KS);
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    separable_pair_f16(av, rb, bv[2 * t], bv[2 * t + 1], kc.one, &h2[t], &l2[t]);
                }
                const half8v ahi = join_half2x4(h2);
                const half8v alo = join_half2x4(l2);
#pragma unroll
                for (int ge = 0; ge < GE; ge++) {
                    acc[r][ge] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bhi[ge], acc[r][ge], 0, 0, 0);
                    acc[r][ge] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, blo[ge], acc[r][ge], 0, 0, 0);
                    acc[r][ge] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bhi[ge], acc[r][ge], 0, 0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        // All reads of the table are done before the next chunk overwrites it.
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
    }

    if (!ok) {
        // Outside the conditions of the feature form: this item in the pairwise form.
        pairwise_item<KT, TL, R>(a, g.x1, g.x2, g.left, g.right, kc, row0, col_begin, col_end, prow);
        return;
    }

    // Row weights of the three sums for every feature, tab_w[row][feature][3], over the column
    // tables (all reads of those are done).  With pw the power of g in the feature and cB / sB its
    // phase factor, (h - g)^2 contributes h^2, -2 h, 1 and (h - g) contributes h, -1, 0 for
    // pw = 0, 1, 2; cos(A - B) = cA cB + sA sB puts cA on the cB features and sA on the sB ones,
    // sin(A - B) = sA cB - cA sB puts sA and -cA there.  Each lane forms the weights of two
    // rows (lane and lane + 64; it holds their coordinates in the A layout: row 16 r + lane % 16).
    float* tab_w = lds;
    {
        const float xa = kk == 0 ? x1v[0] : (kk == 1 ? x1v[1] : (kk == 2 ? x1v[2] : x1v[3]));
        const float xb = kk == 0 ? x1v[4] : (kk == 1 ? x1v[5] : (kk == 2 ? x1v[6] : x1v[7]));
#pragma unroll
        for (int half = 0; half < 2; half++) {
            const float xr = half == 0 ? xa : xb;
            float* w = tab_w + (size_t)(64 * half + lane) * (NF * 3);
            const float h = (xr - c0) * kc.s;
            const float h2 = h * h;
            if (PHASE) {
                const float th = phase_rev(kc.f, xr, c0);
                const float ca = __builtin_amdgcn_cosf(th);
                const float sa = __builtin_amdgcn_sinf(th);
                const float m2h = -2.0f * h;
                w[0] = ca * h2;   w[1] = sa * h;    w[2] = ca;     // cB
                w[3] = sa * h2;   w[4] = -ca * h;   w[5] = sa;     // sB
                w[6] = ca * m2h;  w[7] = -sa;       w[8] = 0.0f;   // cB g
                w[9] = sa * m2h;  w[10] = ca;       w[11] = 0.0f;  // sB g
                w[12] = ca;       w[13] = 0.0f;     w[14] = 0.0f;  // cB g^2
                w[15] = sa;       w[16] = 0.0f;     w[17] = 0.0f;  // sB g^2
            } else {
                w[0] = h2;          w[1] = 1.0f;  w[2] = 0.0f;  // 1
                w[3] = -2.0f * h;   w[4] = 0.0f;  w[5] = 0.0f;  // g
                w[6] = 1.0f;        w[7] = 0.0f;  w[8] = 0.0f;  // g^2
            }
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

    // Accumulators in the D layout: rows 16 r + 4 kk + v, operand column (feature, vector column)
    // of the lane.  Every value times its row's `left` entry and the row weights of its feature.
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
    float unscale[GE];
    const float* wlane[GE];
    const float* llane[GE];
#pragma unroll
    for (int ge = 0; ge < GE; ge++) {
        unscale[ge] = used[ge] ? __builtin_ldexpf(1.0f, -shift[ge] - KS) : 0.0f;
        wlane[ge] = tab_w + (4 * kk) * (NF * 3) + feat[ge] * 3;
        llane[ge] = tab_left + (4 * kk) * a.c + vcol[ge];
    }
#pragma unroll
    for (int r = 0; r < R; r++) {
#pragma unroll
        for (int ge = 0; ge < GE; ge++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const float* w = wlane[ge] + (16 * r + v) * (NF * 3);
                const float lv = llane[ge][(16 * r + v) * a.c];
                const float val = acc[r][ge][v] * unscale[ge] * lv;
                s0 = __builtin_fmaf(w[0], val, s0);
                s1 = __builtin_fmaf(w[1], val, s1);
                if (PHASE) {
                    s2 = __builtin_fmaf(w[2], val, s2);
                }
            }
        }
        // One row group at a time (registers).
        __builtin_amdgcn_sched_barrier(0);
    }
    if (PHASE) {
        s1 *= fabsf(g.params[0]) * (1.0f / KM_SQRT_HALF_LOG2E);  // d = u / s
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    s2 = wave_sum(s2);
    if (lane == 0) {
        prow[0] = s0;
        prow[1] = s1;
        prow[2] = PHASE ? s2 : 0.0f;
        prow[3] = 0.0f;
    }
}

struct ReduceArgs {
    BatchShape batch;
    long long partial_rows;
    const float* partials;
    const float* params;
    BatchStrides params_bs;
    long long params_s;
    float* grad;  // [num_batches][P]
};

#define KM_REDUCE_THREADS 1024

// One workgroup per batch item.  Every thread adds its rows (one 16-byte load each, several in
// flight) in fp64, then a fixed tree over the workgroup: the order of the additions depends on
// the row count alone, so results are reproducible.
template <int KT>
__global__ void __launch_bounds__(KM_REDUCE_THREADS) param_grad_reduce(const ReduceArgs a) {
    constexpr int P = KernelTraits<KT>::P;
    static_assert(KM_MAX_PARAMS == 4, "one float4 per partial row");
    __shared__ double sh[KM_MAX_PARAMS][KM_REDUCE_THREADS];
    const long long b = blockIdx.x;
    const float* __restrict__ base = a.partials + b * a.partial_rows * KM_MAX_PARAMS;
    // (a workspace that is not 16-byte aligned is read one float at a time)
    const bool aligned = ((unsigned long long)base & 15ull) == 0;
    auto load_row = [&](long long r) -> float4v {
        if (aligned) {
            return ((const float4v*)base)[r];
        }
        const float* q = base + r * KM_MAX_PARAMS;
        return (float4v){q[0], q[1], q[2], q[3]};
    };

    double sum[KM_MAX_PARAMS] = {0.0, 0.0, 0.0, 0.0};
    long long i = threadIdx.x;
    for (; i + 3 * KM_REDUCE_THREADS < a.partial_rows; i += 4 * KM_REDUCE_THREADS) {
        float4v v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            v[u] = load_row(i + u * KM_REDUCE_THREADS);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
#pragma unroll
            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                sum[p] += (double)v[u][p];
            }
        }
    }
    for (; i < a.partial_rows; i += KM_REDUCE_THREADS) {
        const float4v v = load_row(i);
#pragma unroll
        for (int p = 0; p < KM_MAX_PARAMS; p++) {
            sum[p] += (double)v[p];
        }
    }
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        sh[p][threadIdx.x] = sum[p];
    }
    __syncthreads();
    for (int half = KM_REDUCE_THREADS / 2; half >= 1; half >>= 1) {
        if ((int)threadIdx.x < half) {
#pragma unroll
            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                sh[p][threadIdx.x] += sh[p][threadIdx.x + half];
            }
        }
        __syncthreads();
    }
    if (threadIdx.x != 0) {
        return;
    }

    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    float* __restrict__ g = a.grad + b * P;
    finish_param_grad<KT>(sh[0][0], sh[1][0], sh[2][0], sh[3][0], params, a.params_s, g);
}

// ---------------------------------------------------------------------------------------
// Host dispatch.
// ---------------------------------------------------------------------------------------
static int grad_col_splits(long long base, bool feature_form = false) {
    // Enough wavefronts to populate the 1024 SIMDs of the device several times over when the
    // row-chunk count alone does not: 4 per SIMD for the pairwise kernels, 2 per SIMD (what fits
    // at its register count) for the feature kernels.  Measured: spectral c = 4, n = 20000,
    // batch 4 (628 row-block items): 36.8 us at 4 column shares against 41.4 us at 7.
    if (base <= 0) {
        return 1;
    }
    const long long target = feature_form ? 2048 : 4096;
    long long s = (target + base - 1) / base;
    if (s < 1) s = 1;
    if (s > 16) s = 16;
    return (int)s;
}

long long param_grad_partials_per_batch(int64_t m, long long num_batches) {
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    return row_blocks * grad_col_splits(row_blocks * num_batches);
}

// Decomposition of the feature form for a vector width c, or GE = 0 when the form does not
// apply (locally periodic kernel, wide vectors).  GE groups of 16 operand columns hold the
// (number of features) x c products; wide operands get fewer rows per wavefront.
struct FeaturePlan {
    int GE, R, TL;
};

static FeaturePlan feature_plan(int kernel_type, int64_t c) {
    FeaturePlan f = {0, 8, 0};
    const int features = kernel_type == KM_KERNEL_SPECTRAL ? 6 : (kernel_type == KM_KERNEL_RBF ? 3 : 0);
    // Up to 32 operand columns: with more, the accumulators leave room for 64 rows per wavefront
    // only, and measured (spectral, c = 8) that is slower than the pairwise form.
    if (features == 0 || c <= 0 || features * c > 32) {
        return f;
    }
    f.GE = (int)((features * c + 15) / 16);
    f.R = 8;
    f.TL = c <= 4 ? 1 : (c <= 8 ? 2 : 4);
    return f;
}

long long param_grad_feature_partials_per_batch(int kernel_type, int64_t m, long long num_batches, int64_t c) {
    const FeaturePlan f = feature_plan(kernel_type, c);
    if (f.GE == 0) {
        return 0;
    }
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    const long long chunks = row_blocks * (8 / f.R);
    return chunks * grad_col_splits(chunks * num_batches, true);
}

void describe_param_grad(int kernel_type, int64_t m, long long num_batches, int64_t c, char* text,
                         size_t text_bytes) {
    static const char* const kernels[] = {"rbf", "spectral", "locally_periodic"};
    const FeaturePlan f = feature_plan(kernel_type, c);
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    const int splits = grad_col_splits(row_blocks * num_batches, f.GE > 0);
    if (f.GE > 0) {
        snprintf(text, text_bytes,
                 "km::param_grad_features<%s, GE=%d, R=%d, TL=%d> (feature form; per-item pairwise fallback) + "
                 "km::param_grad_reduce: 128 rows per wavefront, %d column share(s) per row block",
                 kernels[kernel_type], f.GE, f.R, f.TL, splits);
    } else {
        const int tl = c <= 4 ? 1 : (c <= 8 ? 2 : (c <= 16 ? 4 : 0));
        snprintf(text, text_bytes,
                 "km::param_grad_partial<%s, TL=%d> (pairwise form) + km::param_grad_reduce: 128 rows per "
                 "wavefront, %d column share(s) per row block",
                 kernels[kernel_type], tl, splits);
    }
}

template <int KT, int GE, int R, int TL>
static hipError_t launch_features_as(const GradArgs& a, unsigned grid_x, hipStream_t stream) {
    hipLaunchKernelGGL((param_grad_features<KT, GE, R, TL>), dim3(grid_x), dim3(64),
                       KM_GF_TABLE_FLOATS * sizeof(float), stream, a);
    return hipGetLastError();
}

static hipError_t launch_features(int kernel_type, const FeaturePlan& f, const GradArgs& a, unsigned grid_x,
                                  hipStream_t stream) {
    if (kernel_type == KM_KERNEL_SPECTRAL) {  // 6 features: c <= 5
        if (f.GE == 1) return launch_features_as<KM_KERNEL_SPECTRAL, 1, 8, 1>(a, grid_x, stream);
        if (f.TL == 1) return launch_features_as<KM_KERNEL_SPECTRAL, 2, 8, 1>(a, grid_x, stream);
        return launch_features_as<KM_KERNEL_SPECTRAL, 2, 8, 2>(a, grid_x, stream);
    }
    // rbf, 3 features: c <= 10
    if (f.GE == 1 && f.TL == 1) return launch_features_as<KM_KERNEL_RBF, 1, 8, 1>(a, grid_x, stream);
    if (f.GE == 1) return launch_features_as<KM_KERNEL_RBF, 1, 8, 2>(a, grid_x, stream);
    if (f.TL == 2) return launch_features_as<KM_KERNEL_RBF, 2, 8, 2>(a, grid_x, stream);
    return launch_features_as<KM_KERNEL_RBF, 2, 8, 4>(a, grid_x, stream);
}

// The short addressing and decode of the pairwise kernel apply when the batch shape has
// collapsed to at most one dimension, all counts fit 31 bits and the inner strides are small.
static bool pairwise_fast(const GradArgs& a) {
    const long long limit = 1ll << 31;
    const long long strides[6] = {a.x1_s, a.x2_s, a.left_s0, a.left_s1, a.right_s0, a.right_s1};
    for (long long stride : strides) {
        if (stride < 0 || stride > KM_GRAD_FAST_STRIDE) {
            return false;
        }
    }
    return a.batch.rank <= 1 && a.c >= 1 && a.total_items < limit && a.items_per_xcd * KM_NUM_XCD < limit &&
           a.num_batches < limit;
}

template <int KT, bool FAST>
static hipError_t launch_partial_as(const GradArgs& a, unsigned grid_x, hipStream_t stream) {
    if (a.c <= 4) {
        hipLaunchKernelGGL((param_grad_partial<KT, 1, FAST>), dim3(grid_x), dim3(64), 0, stream, a);
    } else if (a.c <= 8) {
        hipLaunchKernelGGL((param_grad_partial<KT, 2, FAST>), dim3(grid_x), dim3(64), 0, stream, a);
    } else if (a.c <= 16) {
        hipLaunchKernelGGL((param_grad_partial<KT, 4, FAST>), dim3(grid_x), dim3(64), 0, stream, a);
    } else {
        hipLaunchKernelGGL((param_grad_partial<KT, 0, FAST>), dim3(grid_x), dim3(64), 0, stream, a);
    }
    return hipGetLastError();
}

template <int KT>
static hipError_t launch_partial(const GradArgs& a, unsigned grid_x, hipStream_t stream) {
    return pairwise_fast(a) ? launch_partial_as<KT, true>(a, grid_x, stream)
                            : launch_partial_as<KT, false>(a, grid_x, stream);
}

hipError_t launch_param_grad_reduce(int kernel_type, const BatchShape& batch, long long num_batches,
                                    long long partial_rows, const float* partials,
                                    const float* params, const BatchStrides& params_bs,
                                    long long params_s, float* grad, hipStream_t stream) {
    ReduceArgs ra;
    ra.batch = batch;
    ra.partial_rows = partial_rows;
    ra.partials = partials;
    ra.params = params;
    ra.params_bs = params_bs;
    ra.params_s = params_s;
    ra.grad = grad;
    const unsigned rgrid = (unsigned)num_batches;
    switch (kernel_type) {
        case KM_KERNEL_RBF:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_RBF>), dim3(rgrid), dim3(KM_REDUCE_THREADS), 0, stream, ra);
            break;
        case KM_KERNEL_SPECTRAL:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_SPECTRAL>), dim3(rgrid), dim3(KM_REDUCE_THREADS), 0, stream, ra);
            break;
        default:
            hipLaunchKernelGGL((param_grad_reduce<KM_KERNEL_LOCALLY_PERIODIC>), dim3(rgrid), dim3(KM_REDUCE_THREADS), 0, stream, ra);
            break;
    }
    return hipGetLastError();
}

hipError_t launch_param_grad(const ParamGradProblem& p, hipStream_t stream) {
    GradArgs a;
    const int r = p.batch_rank;
    const int64_t* const strides[7] = {p.x1_strides, p.x2_strides, p.left_strides, p.right_strides,
                                       p.params_strides, p.start_strides, p.end_strides};
    BatchStrides* outs[7] = {&a.x1_bs, &a.x2_bs, &a.left_bs, &a.right_bs,
                             &a.params_bs, &a.start_bs, &a.end_bs};
    collapse_batch<7>(r, p.batch_sizes, strides, &a.batch, outs);
    a.num_batches = p.num_batches;
    a.m = (int)p.m;
    a.n = (int)p.n;
    a.c = (int)p.c;
    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    // Feature form where it applies (its 32-bit lane offsets need moderate, non-negative strides
    // of `right`); pairwise form otherwise.
    FeaturePlan fplan = feature_plan(p.kernel_type, p.c);
    {
        const int64_t r0 = p.right_strides[r], r1 = p.right_strides[r + 1];
        if (r0 < 0 || r1 < 0 || r0 > (1 << 24) || r1 > (1 << 24) || p.x2_strides[r] < 0 ||
            p.x2_strides[r] > (1 << 24)) {
            fplan.GE = 0;
        }
    }
    long long chunks = row_blocks;
    if (fplan.GE > 0) {
        chunks = row_blocks * (8 / fplan.R);
    }
    a.col_splits = grad_col_splits(chunks * p.num_batches, fplan.GE > 0);
    a.total_items = chunks * a.col_splits * p.num_batches;
    a.items_per_xcd = (a.total_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    a.partial_rows = chunks * a.col_splits;
    {
        const BatchStrides* const all[7] = {&a.x1_bs, &a.x2_bs, &a.left_bs, &a.right_bs,
                                            &a.params_bs, &a.start_bs, &a.end_bs};
        for (int i = 0; i < 7; i++) {
            a.first_bs[i] = a.batch.rank >= 1 ? all[i]->s[0] : 0;
        }
    }
    a.x1 = p.x1;
    a.x2 = p.x2;
    a.left = p.left;
    a.right = p.right;
    a.params = p.params;
    a.start = p.start;
    a.end = p.end;
    a.partials = (float*)p.workspace;
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.left_s0 = p.left_strides[r];
    a.left_s1 = p.left_strides[r + 1];
    a.right_s0 = p.right_strides[r];
    a.right_s1 = p.right_strides[r + 1];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];

    const unsigned grid_x = (unsigned)(a.items_per_xcd * KM_NUM_XCD);
    if (grid_x > 0 && fplan.GE > 0) {
        const hipError_t err = launch_features(p.kernel_type, fplan, a, grid_x, stream);
        if (err != hipSuccess) {
            return err;
        }
    } else if (grid_x > 0) {  // no rows: the reduce pass alone writes the zero gradient
        hipError_t err;
        switch (p.kernel_type) {
            case KM_KERNEL_RBF: err = launch_partial<KM_KERNEL_RBF>(a, grid_x, stream); break;
            case KM_KERNEL_SPECTRAL: err = launch_partial<KM_KERNEL_SPECTRAL>(a, grid_x, stream); break;
            default: err = launch_partial<KM_KERNEL_LOCALLY_PERIODIC>(a, grid_x, stream); break;
        }
        if (err != hipSuccess) {
            return err;
        }
    }

    return launch_param_grad_reduce(p.kernel_type, a.batch, p.num_batches, chunks * a.col_splits,
                                    a.partials, p.params, a.params_bs, a.params_s, p.grad, stream);
}

}  // namespace km
