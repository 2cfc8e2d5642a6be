// Index operator and its hyper-parameter gradient.
//   index     : out[q] = K[batch_index(q)..., row_index[q], col_index[q]], zero when the
//               column lies outside the row block's [start, end) range
//               (native/index/index.cu:12-101 of the reference).
//   index_bwd : grad[b,p] = d/d params[b,p] sum_{q : batch(q) = b} out_grad[q] * out[q]
//               (native/index_bwd/index_bwd.cu:12-112).  Pass 1 writes the derivative terms of
//               every entry and the batch item it belongs to, and per block of 256 entries their
//               fp64 sums and whether they all belong to one batch item; pass 2 lets one
//               workgroup per batch item add its blocks' sums (the entries themselves only for
//               blocks that mix batch items) in a fixed order and applies the chain rule.
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
    float* terms;     // [total][KM_MAX_PARAMS] (written for the blocks that mix batch items)
    int* owner;       // [total] flat batch item of the entry, -1 if it contributes nothing (likewise)
    int* block_owner;    // [blocks of 256 entries] the one batch item of the block's entries, -1: none
                         // contributes, -2: several batch items (the per-entry arrays decide)
    double* block_sum;   // [blocks][KM_MAX_PARAMS] sums of the block's terms (fixed order)
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
    __shared__ double sh_sum[KM_MAX_PARAMS][256];
    __shared__ int sh_lo[256], sh_hi[256];
    const long long q = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    float acc[KM_MAX_PARAMS] = {0.0f, 0.0f, 0.0f, 0.0f};
    int owner = -1;
    if (q < a.total) {
        const Entry en = decode_entry(a, q);
        if (en.inside) {
            const KernelConsts kc = make_consts<KT>(en.params, a.params_s, false);
            accumulate_pair<KT>(en.x1, en.x2, a.out_grad[en.grad_off], kc, acc);
            owner = (int)en.batch;
        }
    }
    // The block's sums (fixed order) and whether all its contributing entries belong to one
    // batch item: then the second pass takes the sums and never looks at the entries, which are
    // only written for blocks that mix batch items.
#pragma unroll
    for (int p = 0; p < KM_MAX_PARAMS; p++) {
        sh_sum[p][threadIdx.x] = (double)acc[p];
    }
    sh_lo[threadIdx.x] = owner >= 0 ? owner : 0x7fffffff;
    sh_hi[threadIdx.x] = owner;
    __syncthreads();
    for (int half = 128; half >= 1; half >>= 1) {
        if ((int)threadIdx.x < half) {
#pragma unroll
            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                sh_sum[p][threadIdx.x] += sh_sum[p][threadIdx.x + half];
            }
            sh_lo[threadIdx.x] = min(sh_lo[threadIdx.x], sh_lo[threadIdx.x + half]);
            sh_hi[threadIdx.x] = max(sh_hi[threadIdx.x], sh_hi[threadIdx.x + half]);
        }
        __syncthreads();
    }
    const int lo = sh_lo[0], hi = sh_hi[0];
    if (hi >= 0 && lo != hi && q < a.total) {
#pragma unroll
        for (int p = 0; p < KM_MAX_PARAMS; p++) {
            a.terms[q * KM_MAX_PARAMS + p] = acc[p];
        }
        a.owner[q] = owner;
    }
    if (threadIdx.x == 0) {
        a.block_owner[blockIdx.x] = hi < 0 ? -1 : (lo == hi ? lo : -2);
#pragma unroll
        for (int p = 0; p < KM_MAX_PARAMS; p++) {
            a.block_sum[(long long)blockIdx.x * KM_MAX_PARAMS + p] = sh_sum[p][0];
        }
    }
}

template <int KT>
__global__ void __launch_bounds__(256) index_bwd_reduce(const IndexArgs a) {
    constexpr int P = KernelTraits<KT>::P;
    __shared__ double sh[KM_MAX_PARAMS][256];
    const int b = blockIdx.x;
    const long long blocks = (a.total + 255) / 256;
    __shared__ unsigned long long sh_mixed[4][4];  // [quarter][wavefront] which blocks mix batch items
    double sum[KM_MAX_PARAMS] = {0.0, 0.0, 0.0, 0.0};
    // 1024 blocks at a time, four per thread (their loads in flight together): a block of this
    // batch item alone adds its sums; blocks that mix batch items are then gone through by the
    // whole workgroup, one entry per thread.  The order of every thread's additions is fixed.
    const int wave = threadIdx.x >> 6;
    for (long long i0 = 0; i0 < blocks; i0 += 1024) {
        int who[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const long long i = i0 + 256 * u + threadIdx.x;
            who[u] = i < blocks ? a.block_owner[i] : -1;
        }
        bool mixed = false;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            const long long i = i0 + 256 * u + threadIdx.x;
            if (who[u] == b) {
#pragma unroll
                for (int p = 0; p < KM_MAX_PARAMS; p++) {
                    sum[p] += a.block_sum[i * KM_MAX_PARAMS + p];
                }
            }
            mixed = mixed || who[u] == -2;
        }
        if (__syncthreads_or(mixed)) {
#pragma unroll
            for (int u = 0; u < 4; u++) {
                const unsigned long long m = __ballot(who[u] == -2);
                if ((threadIdx.x & 63) == 0) {
                    sh_mixed[u][wave] = m;
                }
            }
            __syncthreads();
            for (int u = 0; u < 4; u++) {
                for (int w = 0; w < 4; w++) {
                    unsigned long long m = sh_mixed[u][w];
                    while (m != 0) {
                        const int j = __builtin_ctzll(m);
                        m &= m - 1;
                        const long long q = (i0 + 256 * u + 64 * w + j) * 256 + threadIdx.x;
                        if (q < a.total && a.owner[q] == b) {
#pragma unroll
                            for (int p = 0; p < KM_MAX_PARAMS; p++) {
                                sum[p] += (double)a.terms[q * KM_MAX_PARAMS + p];
                            }
                        }
                    }
                }
            }
            __syncthreads();
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
    a.block_owner = nullptr;
    a.block_sum = nullptr;
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

// Per entry: KM_MAX_PARAMS terms and the owner; per block of 256 entries: owner and sums.
static size_t index_bwd_entry_bytes(long long total_entries) {
    const size_t bytes = (size_t)total_entries * (KM_MAX_PARAMS * sizeof(float) + sizeof(int));
    return (bytes + 7) & ~(size_t)7;
}

size_t index_bwd_workspace_bytes(long long total_entries) {
    const size_t blocks = (size_t)((total_entries + 255) / 256);
    return index_bwd_entry_bytes(total_entries) + blocks * KM_MAX_PARAMS * sizeof(double) +
           blocks * sizeof(int);
}

hipError_t launch_index_bwd(const IndexBwdProblem& p, hipStream_t stream) {
    IndexArgs a;
    fill_args(a, p.index);
    a.out_grad = p.out_grad;
    fill_index(a.out_grad_strides, p.out_grad_strides, p.index.index_rank);
    a.terms = (float*)p.workspace;
    a.owner = (int*)((char*)p.workspace + (size_t)a.total * KM_MAX_PARAMS * sizeof(float));
    a.block_sum = (double*)((char*)p.workspace + index_bwd_entry_bytes(a.total));
    a.block_owner = (int*)(a.block_sum + (size_t)((a.total + 255) / 256) * KM_MAX_PARAMS);
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
