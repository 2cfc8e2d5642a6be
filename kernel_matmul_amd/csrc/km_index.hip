// Index operator and its hyper-parameter gradient.
//   index     : out[q] = K[batch_index(q)..., row_index[q], col_index[q]], zero when the
//               column lies outside the row block's [start, end) range
//               (native/index/index.cu:12-101 of the reference).
//   index_bwd : grad[b,p] = d/d params[b,p] sum_{q : batch(q) = b} out_grad[q] * out[q]
//               (native/index_bwd/index_bwd.cu:12-112).  Pass 1 writes the derivative terms of
//               every entry and the batch item it belongs to; pass 2 lets one workgroup per
//               batch item add its entries in a fixed order in fp64 and applies the chain rule.
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
    int batch_sizes[KM_MAX_BATCH_RANK];
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
    // index_bwd only
    const float* out_grad;
    IndexStrides out_grad_strides;
    float* terms;     // [total][KM_MAX_PARAMS]
    int* owner;       // [total] flat batch item of the entry, -1 if it contributes nothing
    long long num_batches;
    float* grad;      // [num_batches][P]
};

struct Entry {
    bool inside;        // within the matrix and the sparsity pattern
    long long batch;    // flat batch item
    float x1, x2;
    const float* params;
    long long grad_off;  // position in out_grad
};

__device__ __forceinline__ Entry decode_entry(const IndexArgs& a, long long q) {
    long long rest = q;
    long long row_off = 0, col_off = 0, grad_off = 0;
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
            grad_off += i * a.out_grad_strides.s[d];
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

    Entry en;
    en.grad_off = grad_off;
    en.batch = 0;
    bool batch_ok = true;
    long long x1_off = 0, x2_off = 0, params_off = 0, start_off = 0, end_off = 0;
#pragma unroll
    for (int e = 0; e < KM_MAX_BATCH_RANK; e++) {
        if (e < a.batch_rank) {
            const long long bi = a.batch_index[e][bi_off[e]];
            batch_ok = batch_ok && bi >= 0 && bi < a.batch_sizes[e];
            en.batch = en.batch * a.batch_sizes[e] + bi;
            x1_off += bi * a.x1_bs.s[e];
            x2_off += bi * a.x2_bs.s[e];
            params_off += bi * a.params_bs.s[e];
            start_off += bi * a.start_bs.s[e];
            end_off += bi * a.end_bs.s[e];
        }
    }
    en.inside = false;
    en.x1 = 0.0f;
    en.x2 = 0.0f;
    en.params = a.params + params_off;
    if (batch_ok && row >= 0 && row < a.m && col >= 0 && col < a.n) {
        const int block = row / KM_BLOCK_SIZE;
        const int range_start = a.start[start_off + block * a.start_s];
        const int range_end = a.end[end_off + block * a.end_s];
        if (range_start <= col && col < range_end) {
            en.inside = true;
            en.x1 = a.x1[x1_off + (long long)row * a.x1_s];
            en.x2 = a.x2[x2_off + (long long)col * a.x2_s];
        }
    }
    return en;
}

template <int KT>
__global__ void __launch_bounds__(256) index_kernel(const IndexArgs a) {
    const long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= a.total) {
        return;
    }
    const Entry en = decode_entry(a, q);
    float value = 0.0f;
    if (en.inside) {
        const KernelConsts kc = make_consts<KT>(en.params, a.params_s, true);
        value = kernel_value<KT>(en.x1, en.x2, kc) * kc.sgn;
    }
    a.out[q] = value;
}

template <int KT>
__global__ void __launch_bounds__(256) index_bwd_terms(const IndexArgs a) {
    const long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (q >= a.total) {
        return;
    }
    const Entry en = decode_entry(a, q);
    float acc[KM_MAX_PARAMS] = {0.0f, 0.0f, 0.0f, 0.0f};
    int owner = -1;
    if (en.inside) {
        const KernelConsts kc = make_consts<KT>(en.params, a.params_s, false);
        accumulate_pair<KT>(en.x1, en.x2, a.out_grad[en.grad_off], kc, acc);
        owner = (int)en.batch;
    }
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        a.terms[q * KM_MAX_PARAMS + p] = acc[p];
    }
    a.owner[q] = owner;
}

template <int KT>
__global__ void __launch_bounds__(256) index_bwd_reduce(const IndexArgs a) {
    constexpr int P = KernelTraits<KT>::P;
    __shared__ double sh[KM_MAX_PARAMS][256];
    const int b = blockIdx.x;
    double sum[KM_MAX_PARAMS] = {0.0, 0.0, 0.0, 0.0};
    for (long long q = threadIdx.x; q < a.total; q += 256) {
        if (a.owner[q] == b) {
#pragma unroll
            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                sum[p] += (double)a.terms[q * KM_MAX_PARAMS + p];
            }
        }
    }
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        sh[p][threadIdx.x] = sum[p];
    }
    __syncthreads();
    for (int half = 128; half >= 1; half >>= 1) {
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
    // Parameters of batch item b (row-major flat index over the batch shape).
    long long params_off = 0;
    int rest = b;
#pragma unroll
    for (int e = KM_MAX_BATCH_RANK - 1; e >= 0; e--) {
        if (e < a.batch_rank) {
            params_off += (long long)(rest % a.batch_sizes[e]) * a.params_bs.s[e];
            rest /= a.batch_sizes[e];
        }
    }
    finish_param_grad<KT>(sh[0][0], sh[1][0], sh[2][0], sh[3][0], a.params + params_off, a.params_s,
                          a.grad + (long long)b * P);
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

static void fill_args(IndexArgs& a, const IndexProblem& p) {
    const int r = p.batch_rank;
    a.batch_rank = r;
    for (int d = 0; d < KM_MAX_BATCH_RANK; d++) {
        a.batch_sizes[d] = d < r ? (int)p.batch_sizes[d] : 1;
    }
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
        fill_index(a.batch_index_strides[e], e < r ? p.batch_index_strides[e] : nullptr,
                   e < r ? p.index_rank : 0);
    }
    a.row_index = p.row_index;
    a.col_index = p.col_index;
    fill_index(a.row_strides, p.row_index_strides, p.index_rank);
    fill_index(a.col_strides, p.col_index_strides, p.index_rank);
    a.out = p.out;
    a.out_grad = nullptr;
    fill_index(a.out_grad_strides, nullptr, 0);
    a.terms = nullptr;
    a.owner = nullptr;
    a.num_batches = 0;
    a.grad = nullptr;
}

hipError_t launch_index(const IndexProblem& p, hipStream_t stream) {
    IndexArgs a;
    fill_args(a, p);
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

size_t index_bwd_workspace_bytes(long long total_entries) {
    return (size_t)total_entries * (KM_MAX_PARAMS * sizeof(float) + sizeof(int));
}

hipError_t launch_index_bwd(const IndexBwdProblem& p, hipStream_t stream) {
    IndexArgs a;
    fill_args(a, p.index);
    a.out_grad = p.out_grad;
    fill_index(a.out_grad_strides, p.out_grad_strides, p.index.index_rank);
    a.terms = (float*)p.workspace;
    a.owner = (int*)((char*)p.workspace + (size_t)a.total * KM_MAX_PARAMS * sizeof(float));
    a.num_batches = p.num_batches;
    a.grad = p.grad;
    const int kt = p.index.kernel_type;
    if (a.total > 0) {
        const unsigned grid = (unsigned)((a.total + 255) / 256);
        if (kt == KM_KERNEL_RBF) {
            hipLaunchKernelGGL((index_bwd_terms<KM_KERNEL_RBF>), dim3(grid), dim3(256), 0, stream, a);
        } else if (kt == KM_KERNEL_SPECTRAL) {
            hipLaunchKernelGGL((index_bwd_terms<KM_KERNEL_SPECTRAL>), dim3(grid), dim3(256), 0, stream, a);
        } else {
            hipLaunchKernelGGL((index_bwd_terms<KM_KERNEL_LOCALLY_PERIODIC>), dim3(grid), dim3(256), 0, stream, a);
        }
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) {
            return err;
        }
    }
    if (p.num_batches == 0) {
        return hipSuccess;
    }
    const unsigned rgrid = (unsigned)p.num_batches;
    if (kt == KM_KERNEL_RBF) {
        hipLaunchKernelGGL((index_bwd_reduce<KM_KERNEL_RBF>), dim3(rgrid), dim3(256), 0, stream, a);
    } else if (kt == KM_KERNEL_SPECTRAL) {
        hipLaunchKernelGGL((index_bwd_reduce<KM_KERNEL_SPECTRAL>), dim3(rgrid), dim3(256), 0, stream, a);
    } else {
        hipLaunchKernelGGL((index_bwd_reduce<KM_KERNEL_LOCALLY_PERIODIC>), dim3(rgrid), dim3(256), 0, stream, a);
    }
    return hipGetLastError();
}

}  // namespace km
