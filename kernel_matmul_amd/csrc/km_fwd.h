// Definitions shared by the forward (K @ rhs) kernels.
#pragma once

#include "km_common.h"

namespace km {

typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float2v __attribute__((ext_vector_type(2)));
typedef _Float16 half4v __attribute__((ext_vector_type(4)));

__device__ __forceinline__ half8v join_half2x4(const half2v (&p)[4]) {
    const half4v a = __builtin_shufflevector(p[0], p[1], 0, 1, 2, 3);
    const half4v b = __builtin_shufflevector(p[2], p[3], 0, 1, 2, 3);
    return __builtin_shufflevector(a, b, 0, 1, 2, 3, 4, 5, 6, 7);
}

// Element at a wave-uniform base plus a per-lane offset in BYTES (32 bits).
__device__ __forceinline__ float load_at(const float* uniform_base, unsigned lane_bytes) {
    return *(const float*)((const char*)uniform_base + lane_bytes);
}

// The same through a buffer resource: base and a wave-uniform byte offset in scalar registers,
// the lane's byte offset in one vector register - no 64-bit vector arithmetic per load (the
// compiler forms global addresses with a v_lshl_add_u64 each otherwise).  Raw resource over the
// whole 32-bit offset range: no bounds clamp, offsets stay below 2^32 by the stride limits the
// entry point checks.
typedef __amdgpu_buffer_rsrc_t buffer_rsrc;
__device__ __forceinline__ buffer_rsrc uniform_buffer(const float* uniform_base) {
    // The base is the same in every lane; reading it from the first lane tells the compiler so
    // (a resource it takes for divergent is looped over its distinct values around every load).
    const unsigned long long bits = (unsigned long long)uniform_base;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)bits);
    const unsigned hi = __builtin_amdgcn_readfirstlane((unsigned)(bits >> 32));
    return __builtin_amdgcn_make_buffer_rsrc((void*)(((unsigned long long)hi << 32) | lo), 0, -1, 0x00020000);
}
__device__ __forceinline__ float buffer_at(buffer_rsrc rsrc, unsigned lane_bytes, unsigned uniform_bytes) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)lane_bytes, (int)uniform_bytes, 0));
}

// Launch arguments of the forward kernels (batch dimensions already collapsed).
struct FwdArgs {
    BatchShape batch;
    long long num_batches;
    long long total_items;   // row chunks * batches
    long long items_per_xcd;
    int m, n, k;
    int chunks_per_block;    // 128 / rows per workgroup
    int tail_items;          // per XCD: row-block items at the end that are dispatched last in pieces
                             // (direct kernel: 8 pieces of 16 rows; grouped table kernel: 4 column shares)
    int tail_half_items;     // grouped table kernel: how many of these, the very last, are also cut
                             // into two halves of 64 rows (two workgroups)
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

struct MatmulProblem;
// Collapses the batch dimensions and copies pointers, sizes and strides (item counts are left
// to the caller).
void fill_fwd_args(const MatmulProblem& p, FwdArgs* args);

// The split-fp16 kernels evaluate K / sigma scaled by 2^14 (folded into the exponent of the
// base-2 exponential) so that its hi and lo halves stay inside the fp16 exponent range.
#define KM_F16_KSCALE_LOG2 14

// Phase f * (x - c) in revolutions, reduced to [-0.5, 0.5].  x - c is taken as an unevaluated
// sum hi + lo (error-free transformation) and the product f * hi is never rounded on its own
// (fused multiply-add), so the result carries about half an fp32 ulp of 0.5 (3e-8 revolutions) whatever the
// distance to c — the accuracy of a double-precision evaluation at a third of its cost.
__device__ __forceinline__ float phase_rev(float f, float x, float c) {
    const float hi = x - c;
    const float bb = hi - x;
    const float lo = (x - (hi - bb)) - (c + bb);
    // f * hi - round(f * hi) in one fma (exact product, one rounding of a value within
    // [-0.5, 0.5]), then the contribution of lo.
    const float turns = __builtin_rintf(f * hi);
    return __builtin_fmaf(f, lo, __builtin_fmaf(f, hi, -turns));
}

// fp16 roundings of the residuals a0 * b0 - h[0], a1 * b1 - h[1] of two products against their
// fp16 values h (the low halves of the hi + lo split).  Written as two fp32 results (one
// v_fma_mix_f32 each, reading the fp16 operand directly) rounded together by one
// v_cvt_pk_f16_f32: measured on gfx950, v_fma_mixlo_f16 / v_fma_mixhi_f16, which would round
// inside the fused instruction, issue at half the rate of v_fma_mix_f32, so the two-instruction
// form per value pair costs a fifth more than these three.
__device__ __forceinline__ half2v residual_f16x2(float a0, float b0, float a1, float b1, half2v h) {
    const float2v res = {__builtin_fmaf(a0, b0, -(float)h[0]), __builtin_fmaf(a1, b1, -(float)h[1])};
    return __builtin_convertvector(res, half2v);
}

// Separable form of the Gaussian factor (table kernels): K / sigma is evaluated times
// 2^KM_TABLE_KSCALE_LOG2, and a chunk of columns may take the form only while every scaled
// distance of a column to its reference point stays within KM_TABLE_SPAN.
#define KM_TABLE_KSCALE_LOG2 11
#define KM_TABLE_SPAN 2.0f

// Separable form of the Gaussian factor: 2^(ra * b + rb) for two neighbouring columns, with
// ra * b = 2 a b (the factor 2 carried by either operand), rb = KS - a^2, a = (x1 - r) s the
// row's and b = (x2 - r) s the columns' scaled distances to a common reference point r; times
// the columns' 2^(-b^2) (carried by the rhs operand) this is 2^(KS - ((x1 - x2) s)^2).
__device__ __forceinline__ void separable_pair_f16(float ra, float rb, float ba, float bb, float one,
                                                   half2v* hi, half2v* lo) {
    const float ea = __builtin_amdgcn_exp2f(__builtin_fmaf(ra, ba, rb));
    const float eb = __builtin_amdgcn_exp2f(__builtin_fmaf(ra, bb, rb));
    const float2v kv = {ea, eb};
    const half2v h = __builtin_convertvector(kv, half2v);
    *hi = h;
    *lo = residual_f16x2(ea, one, eb, one, h);
}

// The same with the oscillating factor of the spectral kernel per entry: times the cosine of
// the phase difference (revolutions) between the row and each of the two columns.  The low halves
// are the residuals of the exact products e * cos.
__device__ __forceinline__ void separable_pair_cos_f16(float ra, float rb, float ba, float bb, float pha,
                                                       float phb, half2v* hi, half2v* lo) {
    const float ea = __builtin_amdgcn_exp2f(__builtin_fmaf(ra, ba, rb));
    const float eb = __builtin_amdgcn_exp2f(__builtin_fmaf(ra, bb, rb));
    const float ca = __builtin_amdgcn_cosf(pha);
    const float cb = __builtin_amdgcn_cosf(phb);
    const float2v kv = {ea * ca, eb * cb};
    const half2v h = __builtin_convertvector(kv, half2v);
    *hi = h;
    *lo = residual_f16x2(ea, ca, eb, cb, h);
}

__device__ __forceinline__ void split_f16x8(const float (&v)[8], float one, half8v* hi, half8v* lo) {
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

// Minimum and maximum over the wavefront, returned wave-uniform.  Row-wise DPP steps, then the
// last lane of each row of 16 is carried into the following rows; lane 63 holds the result.
__device__ __forceinline__ void wave_min_max(float* lo, float* hi) {
    float a = *lo, b = *hi;
#define KM_DPP_STEP(ctrl)                                                                              \
    a = fminf(a, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, a),     \
                                                                       __builtin_bit_cast(int, a), ctrl, 0xf, 0xf, false))); \
    b = fmaxf(b, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, b),     \
                                                                       __builtin_bit_cast(int, b), ctrl, 0xf, 0xf, false)))
    KM_DPP_STEP(0xb1);   // quad_perm [1, 0, 3, 2]
    KM_DPP_STEP(0x4e);   // quad_perm [2, 3, 0, 1]
    KM_DPP_STEP(0x114);  // row_shr 4
    KM_DPP_STEP(0x118);  // row_shr 8
    KM_DPP_STEP(0x142);  // row_bcast 15
    KM_DPP_STEP(0x143);  // row_bcast 31
#undef KM_DPP_STEP
    *lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, a), 63));
    *hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, b), 63));
}

// Largest value over the 4 lanes that share an rhs column (lanes l, l+16, l+32, l+48).
__device__ __forceinline__ float column_max(float m) {
    const unsigned bits = __float_as_uint(m);
    const auto rows = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
    m = fmaxf(__uint_as_float(rows[0]), __uint_as_float(rows[1]));
    const unsigned bits2 = __float_as_uint(m);
    const auto halves = __builtin_amdgcn_permlane32_swap(bits2, bits2, false, false);
    return fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}

// Per-wavefront view of the problem, shared by the forward kernels.
struct WaveView {
    long long b;
    int row_block;
    const float* x1;
    const float* x2;
    const float* rhs;
    const float* params;
    int range_start;
    int range_end;
};

// FAST: take the short way when the batch shape has collapsed to at most one dimension (small
// launches, where the scalar prologue is a visible part of a wavefront's life; the large grouped
// launches measure 2 % slower with the extra branch and keep the general code).
template <bool FAST = false>
__device__ __forceinline__ WaveView wave_view(const FwdArgs& a, long long item, int chunks_per_block,
                                              int* chunk_in_block) {
    WaveView w;
    w.b = item % a.num_batches;
    const int chunk = (int)(item / a.num_batches);
    w.row_block = chunk / chunks_per_block;
    *chunk_in_block = chunk % chunks_per_block;
    long long off_x1, off_x2, off_rhs, off_params, off_start, off_end;
    if (FAST && a.batch.rank <= 1) {
        // The usual case after the host has collapsed the batch dimensions: one stride per
        // tensor, no division chain.
        off_x1 = w.b * a.x1_bs.s[0];
        off_x2 = w.b * a.x2_bs.s[0];
        off_rhs = w.b * a.rhs_bs.s[0];
        off_params = w.b * a.params_bs.s[0];
        off_start = w.b * a.start_bs.s[0];
        off_end = w.b * a.end_bs.s[0];
    } else {
        int bidx[KM_MAX_BATCH_RANK];
        batch_multi_index(a.batch, w.b, bidx);
        off_x1 = batch_offset(a.batch, a.x1_bs, bidx);
        off_x2 = batch_offset(a.batch, a.x2_bs, bidx);
        off_rhs = batch_offset(a.batch, a.rhs_bs, bidx);
        off_params = batch_offset(a.batch, a.params_bs, bidx);
        off_start = batch_offset(a.batch, a.start_bs, bidx);
        off_end = batch_offset(a.batch, a.end_bs, bidx);
    }
    w.x1 = a.x1 + off_x1;
    w.x2 = a.x2 + off_x2;
    w.rhs = a.rhs + off_rhs;
    w.params = a.params + off_params;
    // Clamped to the valid columns: a symmetric pattern over fewer points than one block
    // reports end = block size > n (native/ranges/ranges.cpp:82-93 of the reference).
    w.range_start = max(a.start[off_start + w.row_block * a.start_s], 0);
    w.range_end = min(a.end[off_end + w.row_block * a.end_s], a.n);
    return w;
}

// Work item of this workgroup.  Items are (row chunk, batch item) pairs, contiguous ranges of
// which belong to one XCD (see xcd_item).  When the launch has a "tail" (only with 128 rows per
// wavefront), the last `tail_items` items of every XCD are cut into 8 pieces of 16 rows that are
// dispatched last: wavefronts are handed out in order, so these short pieces fill the SIMDs
// that would otherwise idle while others finish a last full-size wavefront.
struct ItemRef {
    bool valid;
    bool small;        // a 16-row piece of a tail item
    long long item;    // (row chunk, batch) index
    int piece;         // which 16-row piece (small only)
};

__device__ __forceinline__ ItemRef decode_item(const FwdArgs& a) {
    ItemRef it;
    it.small = false;
    it.piece = 0;
    if (a.tail_items == 0) {
        it.item = xcd_item(blockIdx.x, a.items_per_xcd);
    } else {
        const unsigned xcd = blockIdx.x % KM_NUM_XCD;
        const long long slot = blockIdx.x / KM_NUM_XCD;
        const long long big = a.items_per_xcd - a.tail_items;
        if (slot < big) {
            it.item = (long long)xcd * a.items_per_xcd + slot;
        } else {
            const long long t = slot - big;
            it.small = true;
            it.item = (long long)xcd * a.items_per_xcd + big + t / 8;
            it.piece = (int)(t % 8);
        }
    }
    it.valid = it.item < a.total_items;
    return it;
}

}  // namespace km
