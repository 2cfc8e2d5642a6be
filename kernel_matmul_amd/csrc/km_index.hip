// Index operator: gathers single entries of the masked kernel matrix.
// Computes what native/index/index.cu:12-57 of the reference computes: one entry per
// thread, zero when the column lies outside the row block's [start, end) range.
#include "km_common.h"
#include "km_launch.h"

namespace km {

struct IndexShape {
    int rank;
    long long sizes[KM_MAX_BATCH_RANK + 1];
};

struct IndexStrides {
    long long s[KM_MAX_BATCH_RANK + 1];
};

struct IndexArgs {
    int batch_rank;
    int m, n;
    long long total;
    IndexShape shape;
    const float* x1;
    const float* x2;
    const float* params;
    const int* start;
    const int* end;
    BatchStrides x1_bs, x2_bs, params_bs, start_bs, end_bs;
    long long x1_s, x2_s, params_s, start_s, end_s;
    const int* batch_index[KM_MAX_BATCH_RANK];
    IndexStrides batch_index_strides[KM_MAX_BATCH_RANK];
    const int* row_index;
    IndexStrides row_strides;
    const int* col_index;
    IndexStrides col_strides;
    float* out;
};

template <int KT>
__global__ void __launch_bounds__(256) index_kernel(const IndexArgs a) {
    const long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= a.total) {
        return;
    }
    // Position inside the index tensors.
    long long rest = q;
    long long row_off = 0, col_off = 0;
    long long bi_off[KM_MAX_BATCH_RANK];
#pragma unroll
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        bi_off[d] = 0;
    }
#pragma unroll
    for (int d = KM_MAX_BATCH_RANK; d >= 0; d--) {
        if (d < a.shape.rank) {
            const long long i = rest % a.shape.sizes[d];
            rest /= a.shape.sizes[d];
            row_off += i * a.row_strides.s[d];
            col_off += i * a.col_strides.s[d];
#pragma unroll
            for (int e = 0; e < KM_MAX_BATCH_RANK; e++) {
                if (e < a.batch_rank) {
                    bi_off[e] += i * a.batch_index_strides[e].s[d];
                }
            }
        }
    }
    const int row = a.row_index[row_off];
    const int col = a.col_index[col_off];

    long long x1_off = 0, x2_off = 0, params_off = 0, start_off = 0, end_off = 0;
#pragma unroll
    for (int e = 0; e < KM_MAX_BATCH_RANK; e++) {
        if (e < a.batch_rank) {
            const long long bi = a.batch_index[e][bi_off[e]];
            x1_off += bi * a.x1_bs.s[e];
            x2_off += bi * a.x2_bs.s[e];
            params_off += bi * a.params_bs.s[e];
            start_off += bi * a.start_bs.s[e];
            end_off += bi * a.end_bs.s[e];
        }
    }

    float value = 0.0f;
    if (row >= 0 && row < a.m && col >= 0 && col < a.n) {
        const int block = row / KM_BLOCK_SIZE;
        const int range_start = a.start[start_off + block * a.start_s];
        const int range_end = a.end[end_off + block * a.end_s];
        if (range_start <= col && col < range_end) {
            const KernelConsts kc = make_consts<KT>(a.params + params_off, a.params_s, true);
            const float x1v = a.x1[x1_off + (long long)row * a.x1_s];
            const float x2v = a.x2[x2_off + (long long)col * a.x2_s];
            value = kernel_value<KT>(x1v, x2v, kc) * kc.sgn;
        }
    }
    a.out[q] = value;
}

static void fill_batch(BatchStrides& dst, const int64_t* strides, int rank) {
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        dst.s[d] = d < rank ? strides[d] : 0;
    }
}

static void fill_index(IndexStrides& dst, const int64_t* strides, int rank) {
    for (int d = 0; d <= KM_MAX_BATCH_RANK; d++) {
        dst.s[d] = d < rank ? strides[d] : 0;
    }
}

hipError_t launch_index(const IndexProblem& p, hipStream_t stream) {
    IndexArgs a;
    const int r = p.batch_rank;
    a.batch_rank = r;
    a.m = (int)p.m;
    a.n = (int)p.n;
    a.shape.rank = p.index_rank;
    a.total = 1;
    for (int d = 0; d <= KM_MAX_BATCH_RANK; d++) {
        a.shape.sizes[d] = d < p.index_rank ? p.index_sizes[d] : 1;
        a.total *= a.shape.sizes[d];
    }
    a.x1 = p.x1;
    a.x2 = p.x2;
    a.params = p.params;
    a.start = p.start;
    a.end = p.end;
    fill_batch(a.x1_bs, p.x1_strides, r);
    fill_batch(a.x2_bs, p.x2_strides, r);
    fill_batch(a.params_bs, p.params_strides, r);
    fill_batch(a.start_bs, p.start_strides, r);
    fill_batch(a.end_bs, p.end_strides, r);
    a.x1_s = p.x1_strides[r];
    a.x2_s = p.x2_strides[r];
    a.params_s = p.params_strides[r];
    a.start_s = p.start_strides[r];
    a.end_s = p.end_strides[r];
    for (int e = 0; e < KM_MAX_BATCH_RANK; e++) {
        a.batch_index[e] = e < r ? p.batch_index[e] : nullptr;
        if (e < r) {
            fill_index(a.batch_index_strides[e], p.batch_index_strides[e], p.index_rank);
        } else {
            fill_index(a.batch_index_strides[e], nullptr, 0);
        }
    }
    a.row_index = p.row_index;
    a.col_index = p.col_index;
    fill_index(a.row_strides, p.row_index_strides, p.index_rank);
    fill_index(a.col_strides, p.col_index_strides, p.index_rank);
    a.out = p.out;
    if (a.total == 0) {
        return hipSuccess;
    }
    const unsigned grid = (unsigned)((a.total + 255) / 256);
    switch (p.kernel_type) {
        case KM_KERNEL_RBF:
            hipLaunchKernelGGL((index_kernel<KM_KERNEL_RBF>), dim3(grid), dim3(256), 0, stream, a);
            break;
        case KM_KERNEL_SPECTRAL:
            hipLaunchKernelGGL((index_kernel<KM_KERNEL_SPECTRAL>), dim3(grid), dim3(256), 0, stream, a);
            break;
        default:
            hipLaunchKernelGGL((index_kernel<KM_KERNEL_LOCALLY_PERIODIC>), dim3(grid), dim3(256), 0, stream, a);
            break;
    }
    return hipGetLastError();
}

}  // namespace km
