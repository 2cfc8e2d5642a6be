// Forward operator, workgroup-shared operand form of the split-fp16 MFMA kernel (large
// problems).  Same contract as the kernels of km_matmul.hip (what native/matmul/matmul.cu:13-157
// of the reference computes); what changes is who prepares the rhs operand.
//
// A workgroup of 4 wavefronts owns up to 4 consecutive 128-row blocks of one batch item.  Their
// column ranges overlap almost entirely, so the workgroup walks the union of the ranges in
// chunks of 256 columns and prepares the MFMA B operand of a chunk ONCE, cooperatively:
//   phase 1  every thread tabulates one column (x2, the scaled coordinate, and for the
//            phase-split spectral form cos B / sin B), loads its share of rhs and records the
//            largest |rhs| per rhs column (LDS atomic max);
//   phase 2  the per-column power-of-two scale is updated from that maximum, rhs (times
//            cos B / sin B) is scaled, split into fp16 hi + lo and written to LDS in the
//            B-operand layout of v_mfma_f32_16x16x32_f16;
//   consume  each wavefront evaluates K for 32 rows of every row block (so that the four
//            wavefronts always have the same amount of work between barriers) against the 32
//            columns of a step and issues the MFMAs with B read back from LDS.
// Per evaluated pair this leaves sub, (mul,) fma, exp2 and the hi/lo split on the VALU; the rhs
// side, which costs a third of the instructions when every wavefront prepares its own operand,
// is amortised over 512 rows.
//
// Folded coordinates: with c the x2 value in the middle of a step, u = (x1 - x2) s is taken as
// fma(x1 - c, s, -[(x2 - c) s]) with the bracket tabulated per column, which saves one
// instruction per pair (x1 - c costs two subtractions per 16 x 32 tile).  A chunk uses this form
// only when it loses nothing: every x2 - c of the chunk and every x1 - c of the workgroup's rows
// must be exact in fp32 (checked per column by an error-free transformation, for the rows through
// the spread of all coordinates involved) and |(x2 - c) s| must stay below 16, so that the one
// rounding of the tabulated product is below 1e-6 and varies from column to column.  Otherwise
// (coordinates next to the origin, unsorted columns) the chunk takes u = (x1 - x2) s.  The
// decision is uniform for the workgroup.
#include "km_batch.h"
#include "km_common.h"
#include "km_fwd.h"
#include "km_launch.h"

namespace km {

#define KM_BLK_WAVES 4
#define KM_BLK_THREADS (64 * KM_BLK_WAVES)
#define KM_BLK_CHUNK 256                       /* columns per chunk = one per thread */
#define KM_BLK_STEPS (KM_BLK_CHUNK / 32)
#define KM_BLK_ROW_BLOCKS 4                    /* row blocks per (full) workgroup */
#define KM_BLK_FOLD_SPAN 16.0f

// Order-preserving map from float to unsigned (for integer atomic min / max) and back.
__device__ __forceinline__ unsigned float_key(float x) {
    const unsigned b = __float_as_uint(x);
    return b ^ ((b >> 31) ? 0xffffffffu : 0x80000000u);
}
__device__ __forceinline__ float key_float(unsigned k) {
    return __uint_as_float(k ^ ((k >> 31) ? 0x80000000u : 0xffffffffu));
}

struct BlockArgs {
    FwdArgs f;
    long long main_items;     // (group of row blocks, batch item) pairs
    long long main_per_xcd;
    long long tail_items;     // (single row block, batch item) pairs, dispatched last
    long long tail_per_xcd;
    int main_row_blocks;      // row blocks covered by the main items
};

__device__ __forceinline__ void read8(const float* p, float (&dst)[8]) {
    const float4v a = *(const float4v*)p;
    const float4v b = *(const float4v*)(p + 4);
#pragma unroll
    for (int u = 0; u < 4; u++) {
        dst[u] = a[u];
        dst[4 + u] = b[u];
    }
}

__device__ __forceinline__ void split8(const float (&v)[8], float one, half8v* hi, half8v* lo) {
    half2v h2[4], l2[4];
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const float2v p = {v[2 * t], v[2 * t + 1]};
        h2[t] = __builtin_convertvector(p, half2v);
        l2[t] = residual_f16x2(v[2 * t], one, v[2 * t + 1], one, h2[t]);
    }
    *hi = join_half2x4(h2);
    *lo = join_half2x4(l2);
}

// K entries of 2 x 16 rows (row block J of the workgroup) against the 32 columns of a step,
// split into hi / lo halves, and the MFMAs with the step's B operands.
//   FOLD   : xa = x1 - c, x2a = (x2 - c) s, pa / x2p = phases in revolutions
//   !FOLD  : xa = x1, x2a = x2 (pa, x2p unused)
//   MASKED : columns whose bit in `keep` is clear contribute nothing (partial steps at the ends
//            of this row block's range)
template <int KT, bool PHASE, bool FOLD, bool MASKED, int GE, int J>
__device__ __forceinline__ void block_eval(const float (&xa)[2], const float (&pa)[2],
                                           const float (&x2a)[8], const float (&x2p)[8],
                                           unsigned keep, const KernelConsts& kc,
                                           const half8v (&bhi)[GE], const half8v (&blo)[GE],
                                           float4v (&acc)[2 * KM_BLK_ROW_BLOCKS][GE]) {
    constexpr bool COS = KT == KM_KERNEL_SPECTRAL && !PHASE;
    constexpr bool SIN = KT == KM_KERNEL_LOCALLY_PERIODIC;
#pragma unroll
    for (int q = 0; q < 2; q++) {
        const int r = 2 * J + q;
        half2v h2[4], l2[4];
#pragma unroll
        for (int t2 = 0; t2 < 4; t2++) {
            float ea[2], ca[2];
#pragma unroll
            for (int h = 0; h < 2; h++) {
                const int t = 2 * t2 + h;
                const float d = xa[q] - x2a[t];
                const float u = FOLD ? __builtin_fmaf(xa[q], kc.s, -x2a[t]) : d * kc.s;
                const float arg = __builtin_fmaf(-u, u, (float)KM_F16_KSCALE_LOG2);
                ca[h] = 1.0f;
                if (COS) {
                    ea[h] = __builtin_amdgcn_exp2f(arg);
                    ca[h] = __builtin_amdgcn_cosf(FOLD ? pa[q] - x2p[t] : d * kc.f);
                } else if (SIN) {
                    const float sn = __builtin_amdgcn_sinf(FOLD ? pa[q] - x2p[t] : d * kc.f);
                    const float wv = sn * kc.cl;
                    ea[h] = __builtin_amdgcn_exp2f(__builtin_fmaf(-wv, sn, arg));
                } else {
                    ea[h] = __builtin_amdgcn_exp2f(arg);
                }
                if (MASKED && !((keep >> t) & 1u)) {
                    ea[h] = 0.0f;
                    ca[h] = 0.0f;
                }
            }
            const float2v kv = {COS ? ea[0] * ca[0] : ea[0], COS ? ea[1] * ca[1] : ea[1]};
            h2[t2] = __builtin_convertvector(kv, half2v);
            // Residuals of the exact products (fused, reading the fp16 halves directly).
            l2[t2] = residual_f16x2(ea[0], COS ? ca[0] : kc.one, ea[1], COS ? ca[1] : kc.one, h2[t2]);
        }
        const half8v ahi = join_half2x4(h2);
        const half8v alo = join_half2x4(l2);
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, bhi[g], acc[r][g], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi, blo[g], acc[r][g], 0, 0, 0);
        }
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo, bhi[g], acc[r][g], 0, 0, 0);
        }
    }
}

// LDS of one workgroup.
template <int GE>
struct BlockLds {
    float tab[2][4][KM_BLK_CHUNK];        // [parity][x2, (x2 - c) s, cos B | phase, sin B][column]
    float cst[2][KM_BLK_STEPS];           // [parity][step]: reference point c of the step
    half8v bop[KM_BLK_STEPS][GE][2][64];  // [step][group][hi, lo][lane]
    unsigned maxbuf[2][32];               // [parity][rhs column]: bits of max |rhs|
    unsigned nofold[2];                   // [parity]: nonzero if a column forbids the folded form
    unsigned x1lo, x1hi;                  // ordered keys of min / max x1 over the workgroup's rows
};

// One step (32 columns) of row block J for this wavefront's 32 rows.
template <int KT, bool PHASE, bool FOLD, bool MASKED, int G, int J>
__device__ __forceinline__ void block_step(BlockLds<(PHASE ? 2 : 1) * G>& lds, int parity, int chunk0,
                                           int st, int range_start, int range_end,
                                           const float (&x1v)[2 * KM_BLK_ROW_BLOCKS],
                                           const float (&ph1)[2 * KM_BLK_ROW_BLOCKS],
                                           const KernelConsts& kc, int kk, int lane,
                                           float4v (&acc)[2 * KM_BLK_ROW_BLOCKS][(PHASE ? 2 : 1) * G]) {
    constexpr int GE = (PHASE ? 2 : 1) * G;
    constexpr bool TWO = KT != KM_KERNEL_RBF && !PHASE;
    float x2a[8], x2p[8];
    read8(&lds.tab[parity][FOLD ? 1 : 0][32 * st + 8 * kk], x2a);
    if (TWO && FOLD) {
        read8(&lds.tab[parity][2][32 * st + 8 * kk], x2p);
    } else {
#pragma unroll
        for (int t = 0; t < 8; t++) {
            x2p[t] = 0.0f;
        }
    }
    half8v bhi[GE], blo[GE];
#pragma unroll
    for (int g = 0; g < GE; g++) {
        bhi[g] = lds.bop[st][g][0][lane];
        blo[g] = lds.bop[st][g][1][lane];
    }
    const float c = FOLD ? lds.cst[parity][st] : 0.0f;
    const float xa[2] = {x1v[2 * J] - c, x1v[2 * J + 1] - c};
    const float pa[2] = {ph1[2 * J], ph1[2 * J + 1]};
    unsigned keep = 0xffu;
    if (MASKED) {
        keep = 0;
#pragma unroll
        for (int t = 0; t < 8; t++) {
            const int col = chunk0 + 32 * st + 8 * kk + t;
            keep |= (col >= range_start && col < range_end) ? (1u << t) : 0u;
        }
    }
    block_eval<KT, PHASE, FOLD, MASKED, GE, J>(xa, pa, x2a, x2p, keep, kc, bhi, blo, acc);
}

// All steps of the current chunk for row block J: the (at most two) steps that straddle an end
// of the block's column range go through the masked form, the others through a loop without
// masks or branches.  Without folded coordinates (rare) every step takes the masked form.
template <int KT, bool PHASE, bool FOLD, int G, int J>
__device__ __forceinline__ void block_consume_rows(
    BlockLds<(PHASE ? 2 : 1) * G>& lds, int parity, int chunk0, int chunk_end, int range_start,
    int range_end, const float (&x1v)[2 * KM_BLK_ROW_BLOCKS], const float (&ph1)[2 * KM_BLK_ROW_BLOCKS],
    const KernelConsts& kc, int kk, int lane, float4v (&acc)[2 * KM_BLK_ROW_BLOCKS][(PHASE ? 2 : 1) * G]) {
    const int lo = max(range_start, chunk0);
    const int hi = min(range_end, chunk_end);
    if (lo >= hi) {
        return;
    }
    int first = (lo - chunk0) >> 5;
    int last = (hi - 1 - chunk0) >> 5;
    if (!FOLD) {
        for (int st = first; st <= last; st++) {
            block_step<KT, PHASE, false, true, G, J>(lds, parity, chunk0, st, range_start, range_end, x1v,
                                                     ph1, kc, kk, lane, acc);
        }
        return;
    }
    int partial0 = -1, partial1 = -1;
    if (chunk0 + 32 * first < range_start || chunk0 + 32 * first + 32 > range_end) {
        partial0 = first++;
    }
    if (last >= first && chunk0 + 32 * last + 32 > range_end) {
        partial1 = last--;
    }
    for (int i = 0; i < 2; i++) {
        const int st = i == 0 ? partial0 : partial1;
        if (st >= 0) {
            block_step<KT, PHASE, FOLD, true, G, J>(lds, parity, chunk0, st, range_start, range_end, x1v, ph1,
                                                    kc, kk, lane, acc);
        }
    }
    for (int st = first; st <= last; st++) {
        block_step<KT, PHASE, FOLD, false, G, J>(lds, parity, chunk0, st, range_start, range_end, x1v, ph1,
                                                 kc, kk, lane, acc);
    }
}

template <int KT, bool PHASE, bool FOLD, int G>
__device__ __forceinline__ void block_consume(
    BlockLds<(PHASE ? 2 : 1) * G>& lds, int parity, int chunk0, int chunk_end,
    const int (&ws)[KM_BLK_ROW_BLOCKS], const int (&we)[KM_BLK_ROW_BLOCKS],
    const float (&x1v)[2 * KM_BLK_ROW_BLOCKS], const float (&ph1)[2 * KM_BLK_ROW_BLOCKS],
    const KernelConsts& kc, int kk, int lane,
    float4v (&acc)[2 * KM_BLK_ROW_BLOCKS][(PHASE ? 2 : 1) * G]) {
    // Row blocks the workgroup does not have carry empty ranges.
    block_consume_rows<KT, PHASE, FOLD, G, 0>(lds, parity, chunk0, chunk_end, ws[0], we[0], x1v, ph1, kc, kk, lane, acc);
    block_consume_rows<KT, PHASE, FOLD, G, 1>(lds, parity, chunk0, chunk_end, ws[1], we[1], x1v, ph1, kc, kk, lane, acc);
    block_consume_rows<KT, PHASE, FOLD, G, 2>(lds, parity, chunk0, chunk_end, ws[2], we[2], x1v, ph1, kc, kk, lane, acc);
    block_consume_rows<KT, PHASE, FOLD, G, 3>(lds, parity, chunk0, chunk_end, ws[3], we[3], x1v, ph1, kc, kk, lane, acc);
}

template <int KT, bool PHASE, int G>
__global__ void __launch_bounds__(KM_BLK_THREADS, 3) fwd_block(const BlockArgs ba) {
    constexpr int GE = (PHASE ? 2 : 1) * G;
    constexpr int NB = KM_BLK_ROW_BLOCKS;
    constexpr bool TWO = KT != KM_KERNEL_RBF && !PHASE;
    extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
    BlockLds<GE>& lds = *reinterpret_cast<BlockLds<GE>*>(lds_raw);
    const FwdArgs& a = ba.f;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int li = lane & 15;
    const int kk = lane >> 4;
    const int kbase = blockIdx.y * (16 * G);

    // Work item: consecutive items of an XCD share x2 / rhs windows in its L2.  Main items are
    // groups of 4 row blocks; the row blocks after them are tail items of one row block each,
    // dispatched last so that the final round of workgroups is made of short ones.
    long long b;
    int rb0, nblk;
    {
        const unsigned xcd = blockIdx.x % KM_NUM_XCD;
        const long long slot = blockIdx.x / KM_NUM_XCD;
        if (slot < ba.main_per_xcd) {
            const long long item = (long long)xcd * ba.main_per_xcd + slot;
            if (item >= ba.main_items) {
                return;
            }
            b = item % a.num_batches;
            rb0 = (int)(item / a.num_batches) * NB;
            nblk = min(NB, ba.main_row_blocks - rb0);
        } else {
            const long long item = (long long)xcd * ba.tail_per_xcd + (slot - ba.main_per_xcd);
            if (item >= ba.tail_items) {
                return;
            }
            b = item % a.num_batches;
            rb0 = ba.main_row_blocks + (int)(item / a.num_batches);
            nblk = 1;
        }
    }
    int bidx[KM_MAX_BATCH_RANK];
    batch_multi_index(a.batch, b, bidx);
    const float* __restrict__ x1 = a.x1 + batch_offset(a.batch, a.x1_bs, bidx);
    const float* __restrict__ x2 = a.x2 + batch_offset(a.batch, a.x2_bs, bidx);
    // The rhs column offset of this workgroup goes into the 64-bit base so that the 32-bit lane
    // offsets below span at most 24 rows and 16 G columns.
    const float* __restrict__ rhs = a.rhs + batch_offset(a.batch, a.rhs_bs, bidx) + (long long)kbase * a.rhs_s1;
    const float* __restrict__ params = a.params + batch_offset(a.batch, a.params_bs, bidx);
    const int* __restrict__ start = a.start + batch_offset(a.batch, a.start_bs, bidx);
    const int* __restrict__ end = a.end + batch_offset(a.batch, a.end_bs, bidx);

    // Column ranges of the row blocks (clamped to the valid columns: a symmetric pattern over
    // fewer points than one block reports end = block size > n, native/ranges/ranges.cpp:82-93)
    // and their union.
    int ws[NB], we[NB];
    int u0 = a.n, u1 = 0;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        ws[j] = 0;
        we[j] = 0;
        if (j < nblk) {
            ws[j] = max(start[(long long)(rb0 + j) * a.start_s], 0);
            we[j] = min(end[(long long)(rb0 + j) * a.end_s], a.n);
            if (ws[j] < we[j]) {
                u0 = min(u0, ws[j]);
                u1 = max(u1, we[j]);
            } else {
                ws[j] = 0;
                we[j] = 0;
            }
        }
    }

    const KernelConsts kc = make_consts<KT>(params, a.params_s, false);
    const float sigma = params[KernelTraits<KT>::SIGMA * a.params_s];
    // Reference point of the phases (any point near the rows does).
    const float c_ref = x1[(long long)min(rb0 * KM_BLOCK_SIZE + nblk * (KM_BLOCK_SIZE / 2), a.m - 1) * a.x1_s];

    if (tid < 64) {
        lds.maxbuf[tid >> 5][tid & 31] = 0u;
    }
    if (tid < 2) {
        lds.nofold[tid] = 0u;
    }
    if (tid == 2) {
        lds.x1lo = 0xffffffffu;
        lds.x1hi = 0u;
    }
    __syncthreads();

    // Rows of this wavefront: rows 32 wave .. 32 wave + 31 of every row block, as 2 groups of 16.
    float x1v[2 * NB], ph1[2 * NB];
    {
        float lo = __builtin_inff(), hi = -__builtin_inff();
        bool bad = false;
#pragma unroll
        for (int r = 0; r < 2 * NB; r++) {
            const int row = min((rb0 + r / 2) * KM_BLOCK_SIZE + 32 * wave + 16 * (r & 1) + li, a.m - 1);
            x1v[r] = x1[(long long)row * a.x1_s];
            ph1[r] = TWO ? phase_rev(kc.f, x1v[r], c_ref) : 0.0f;
            if (r / 2 < nblk) {
                lo = fminf(lo, x1v[r]);
                hi = fmaxf(hi, x1v[r]);
                bad = bad || x1v[r] != x1v[r];
            }
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            lo = fminf(lo, __shfl_xor(lo, off, 64));
            hi = fmaxf(hi, __shfl_xor(hi, off, 64));
        }
        if (__any(bad)) {
            lo = __builtin_nanf("");  // NaN coordinates: never fold
        }
        if (lane == 0) {
            atomicMin(&lds.x1lo, lo == lo ? float_key(lo) : 0u);
            atomicMax(&lds.x1hi, lo == lo ? float_key(hi) : 0xffffffffu);
        }
    }

    int shift[G];
    float scale[G];
    unsigned rhs_lane[G];
#pragma unroll
    for (int g = 0; g < G; g++) {
        shift[g] = 100;
        scale[g] = __builtin_ldexpf(1.0f, 100);
        rhs_lane[g] = (unsigned)(8 * kk * a.rhs_s0 + (min(kbase + 16 * g + li, a.k - 1) - kbase) * a.rhs_s1);
    }
    float4v acc[2 * NB][GE];
#pragma unroll
    for (int r = 0; r < 2 * NB; r++) {
#pragma unroll
        for (int g = 0; g < GE; g++) {
            acc[r][g] = (float4v){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }

    int parity = 0;
    for (int chunk0 = u0; chunk0 < u1; chunk0 += KM_BLK_CHUNK) {
        const int chunk_end = min(chunk0 + KM_BLK_CHUNK, u1);
        bool wanted = false;
#pragma unroll
        for (int j = 0; j < NB; j++) {
            wanted = wanted || (ws[j] < chunk_end && we[j] > chunk0);
        }
        if (!wanted) {
            continue;  // a gap between the ranges of the row blocks
        }

        // ---- phase 1: column tables, rhs into registers, maxima -------------------------
        {
            const int col = chunk0 + tid;
            const bool valid = col < chunk_end;
            const float xv = x2[(long long)min(col, chunk_end - 1) * a.x2_s];
            // Reference point of this column's step: the x2 value in the middle of the step.
            const float cs = x2[(long long)min(chunk0 + (tid & ~31) + 16, chunk_end - 1) * a.x2_s];
            const float xd = xv - cs;
            const float bb = xd - xv;
            const float err = (xv - (xd - bb)) - (cs + bb);  // exact error of xd (error-free transformation)
            const float xs = xd * kc.s;
            lds.tab[parity][0][tid] = xv;
            lds.tab[parity][1][tid] = xs;
            if ((tid & 31) == 0) {
                lds.cst[parity][tid >> 5] = cs;
            }
            if (PHASE) {
                const float th = phase_rev(kc.f, xv, c_ref);
                lds.tab[parity][2][tid] = valid ? __builtin_amdgcn_cosf(th) : 0.0f;
                lds.tab[parity][3][tid] = valid ? __builtin_amdgcn_sinf(th) : 0.0f;
            } else if (TWO) {
                lds.tab[parity][2][tid] = phase_rev(kc.f, xv, c_ref);
            }
            const bool ok = err == 0.0f && fabsf(xs) <= KM_BLK_FOLD_SPAN;
            if (!__all(ok) && lane == 0) {
                atomicOr(&lds.nofold[parity], 1u);
            }
        }
        float raw[2][G][8];
        if (chunk0 + KM_BLK_CHUNK <= chunk_end) {
            // Full chunk: wave-uniform base (scalar registers) plus a loop-invariant lane offset.
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const float* ru = rhs + (long long)(chunk0 + 32 * (wave + KM_BLK_WAVES * i)) * a.rhs_s0;
#pragma unroll
                for (int t = 0; t < 8; t++) {
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        raw[i][g][t] = (ru + t * a.rhs_s0)[rhs_lane[g]];
                    }
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const int st = wave + KM_BLK_WAVES * i;
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const int row = chunk0 + 32 * st + 8 * kk + t;
                    const float* p = rhs + (long long)min(row, chunk_end - 1) * a.rhs_s0;
#pragma unroll
                    for (int g = 0; g < G; g++) {
                        const float v = p[rhs_lane[g] - (unsigned)(8 * kk * a.rhs_s0)];
                        raw[i][g][t] = row < chunk_end ? v : 0.0f;
                    }
                }
            }
        }
#pragma unroll
        for (int g = 0; g < G; g++) {
            // Largest finite magnitude: infinities and NaNs propagate through the product on
            // their own and must not decide the scale of the finite values.
            float m = 0.0f;
#pragma unroll
            for (int i = 0; i < 2; i++) {
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    const float av = fabsf(raw[i][g][t]);
                    m = fmaxf(m, av < __builtin_inff() ? av : 0.0f);
                }
            }
            m = column_max(m);
            if (kk == 0) {
                atomicMax(&lds.maxbuf[parity][16 * g + li], __float_as_uint(m));
            }
        }
        __syncthreads();

        // ---- phase 2: fold decision, scales, B operand into LDS --------------------------
        bool fold;
        {
            // Every x1 - c is exact if all coordinates involved are multiples of a common
            // power of two q with spread / q < 2^24; q = ulp of the smallest magnitude, so
            // spread <= smallest magnitude (same sign throughout) is sufficient.
            float cs8[8];
            read8(&lds.cst[parity][0], cs8);
            float lo = key_float(lds.x1lo), hi = key_float(lds.x1hi);
#pragma unroll
            for (int t = 0; t < 8; t++) {
                lo = fminf(lo, cs8[t]);
                hi = fmaxf(hi, cs8[t]);
            }
            const bool rows_ok = (lo > 0.0f || hi < 0.0f) && (hi - lo) <= fminf(fabsf(lo), fabsf(hi));
            fold = __builtin_amdgcn_readfirstlane((rows_ok && lds.nofold[parity] == 0u) ? 1 : 0) != 0;
        }
        bool rescale = false;
        float factor[G];
#pragma unroll
        for (int g = 0; g < G; g++) {
            const float mx = __uint_as_float(lds.maxbuf[parity][16 * g + li]);
            const bool grow = !(mx * scale[g] < 32768.0f);
            // mx < 2^e, so mx * 2^(14 - e) < 2^14.
            const int e = __builtin_amdgcn_frexp_expf(mx);
            const int new_shift = grow ? min(max(KM_F16_KSCALE_LOG2 - e, -100), 100) : shift[g];
            factor[g] = __builtin_ldexpf(1.0f, new_shift - shift[g]);
            shift[g] = new_shift;
            scale[g] = __builtin_ldexpf(1.0f, new_shift);
            rescale = rescale || grow;
        }
        if (tid < 32) {
            lds.maxbuf[parity ^ 1][tid] = 0u;
        }
        if (tid == 32) {
            lds.nofold[parity ^ 1] = 0u;
        }
        if (__any(rescale)) {
#pragma unroll
            for (int r = 0; r < 2 * NB; r++) {
#pragma unroll
                for (int g = 0; g < GE; g++) {
                    acc[r][g] *= factor[g % G];
                }
            }
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
            const int st = wave + KM_BLK_WAVES * i;
            float cb[8], sb[8];
            if (PHASE) {
                read8(&lds.tab[parity][2][32 * st + 8 * kk], cb);
                read8(&lds.tab[parity][3][32 * st + 8 * kk], sb);
            }
#pragma unroll
            for (int g = 0; g < G; g++) {
                float v[8];
#pragma unroll
                for (int t = 0; t < 8; t++) {
                    v[t] = raw[i][g][t] * scale[g];
                }
                if (PHASE) {
                    float vc[8], vs[8];
#pragma unroll
                    for (int t = 0; t < 8; t++) {
                        vc[t] = v[t] * cb[t];
                        vs[t] = v[t] * sb[t];
                    }
                    half8v hi, lo;
                    split8(vc, kc.one, &hi, &lo);
                    lds.bop[st][g][0][lane] = hi;
                    lds.bop[st][g][1][lane] = lo;
                    split8(vs, kc.one, &hi, &lo);
                    lds.bop[st][G + g][0][lane] = hi;
                    lds.bop[st][G + g][1][lane] = lo;
                } else {
                    half8v hi, lo;
                    split8(v, kc.one, &hi, &lo);
                    lds.bop[st][g][0][lane] = hi;
                    lds.bop[st][g][1][lane] = lo;
                }
            }
        }
        __syncthreads();

        // ---- consume ---------------------------------------------------------------------
        if (fold) {
            block_consume<KT, PHASE, true, G>(lds, parity, chunk0, chunk_end, ws, we, x1v, ph1, kc, kk, lane, acc);
        } else {
            block_consume<KT, PHASE, false, G>(lds, parity, chunk0, chunk_end, ws, we, x1v, ph1, kc, kk, lane, acc);
        }
        parity ^= 1;
    }

    // ---- epilogue: undo the scales, apply sigma (and cos A / sin A), store ---------------
    float* __restrict__ out = a.out + b * (long long)a.m * a.k;
#pragma unroll
    for (int r = 0; r < 2 * NB; r++) {
        if (r / 2 >= nblk) {
            continue;
        }
        const int row_base = (rb0 + r / 2) * KM_BLOCK_SIZE + 32 * wave + 16 * (r & 1) + 4 * kk;
        // cos A / sin A: formed once per row by the lane that holds the row's coordinate
        // (x1v: row 16 (r & 1) + lane % 16 of the 32), fetched across lanes into the accumulator
        // layout (rows 4 (lane / 16) + v).
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
            const float unscale = __builtin_ldexpf(sigma, -shift[g] - KM_F16_KSCALE_LOG2);
            const int c = kbase + 16 * g + li;
#pragma unroll
            for (int v = 0; v < 4; v++) {
                float res;
                if (PHASE) {
                    res = ca[v] * (acc[r][g][v] * unscale) + sa[v] * (acc[r][G + g][v] * unscale);
                } else {
                    res = acc[r][g][v] * unscale;
                }
                const int row = row_base + v;
                if (row < a.m && c < a.k) {
                    out[(long long)row * a.k + c] = res;
                }
            }
        }
    }
}

template <int KT, bool PHASE, int G>
static hipError_t launch_block_kernel(const BlockArgs& ba, unsigned gx, unsigned gy, hipStream_t stream) {
    constexpr int GE = (PHASE ? 2 : 1) * G;
    hipLaunchKernelGGL((fwd_block<KT, PHASE, G>), dim3(gx, gy, 1), dim3(KM_BLK_THREADS, 1, 1),
                       sizeof(BlockLds<GE>), stream, ba);
    return hipGetLastError();
}

hipError_t launch_matmul_block(const MatmulProblem& p, const MatmulPlan& plan, hipStream_t stream) {
    BlockArgs ba;
    fill_fwd_args(p, &ba.f);
    const long long nb = p.num_batches;
    const int row_blocks = (int)((p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE);
    const long long groups_all = (row_blocks + KM_BLK_ROW_BLOCKS - 1) / KM_BLK_ROW_BLOCKS;

    // Tail balancing: workgroups are handed out in order and `resident` of them run at a time.
    // Full rounds are made of 4-row-block workgroups; the row blocks left over after the last
    // full round become single-row-block workgroups (a quarter of the work each, same 4
    // wavefronts), so the final, partly filled round is short.
    int tail_blocks = 0;
    if (plan.tail_balance) {
        const long long resident = 256LL * 3;
        const long long rounds = groups_all * nb / resident;
        if (rounds >= 1) {
            const long long main_groups = rounds * resident / nb;
            tail_blocks = (int)max(0LL, (long long)row_blocks - main_groups * KM_BLK_ROW_BLOCKS);
        }
    }
    ba.main_row_blocks = row_blocks - tail_blocks;
    const long long main_groups = (ba.main_row_blocks + KM_BLK_ROW_BLOCKS - 1) / KM_BLK_ROW_BLOCKS;
    ba.main_items = main_groups * nb;
    ba.main_per_xcd = (ba.main_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    ba.tail_items = (long long)tail_blocks * nb;
    ba.tail_per_xcd = (ba.tail_items + KM_NUM_XCD - 1) / KM_NUM_XCD;
    const unsigned gx = (unsigned)((ba.main_per_xcd + ba.tail_per_xcd) * KM_NUM_XCD);
    const unsigned gy = (unsigned)((p.k + plan.k_chunk - 1) / plan.k_chunk);
    const int G = plan.k_chunk / 16;
    const bool phase = plan.phase_split != 0;

    switch (p.kernel_type) {
        case KM_KERNEL_RBF:
            return G == 2 ? launch_block_kernel<KM_KERNEL_RBF, false, 2>(ba, gx, gy, stream)
                          : launch_block_kernel<KM_KERNEL_RBF, false, 1>(ba, gx, gy, stream);
        case KM_KERNEL_SPECTRAL:
            if (phase) {
                return launch_block_kernel<KM_KERNEL_SPECTRAL, true, 1>(ba, gx, gy, stream);
            }
            return G == 2 ? launch_block_kernel<KM_KERNEL_SPECTRAL, false, 2>(ba, gx, gy, stream)
                          : launch_block_kernel<KM_KERNEL_SPECTRAL, false, 1>(ba, gx, gy, stream);
        default:
            return G == 2 ? launch_block_kernel<KM_KERNEL_LOCALLY_PERIODIC, false, 2>(ba, gx, gy, stream)
                          : launch_block_kernel<KM_KERNEL_LOCALLY_PERIODIC, false, 1>(ba, gx, gy, stream);
    }
}

}  // namespace km
