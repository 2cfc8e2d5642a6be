// Sparsity pattern ("ranges") builders.
//
// Host functions: sequential two-pointer scans with exactly the comparison semantics of the
// reference (native/ranges/ranges.cpp:8-62, 64-101, 103-150): every test is an fp32
// subtract followed by an fp32 compare against the fp32 cutoff.
//
// Device functions: the same results for ascending inputs, computed without leaving the
// GPU.  For sorted x the scan predicates are monotone along a row and their first-true
// positions are monotone from row block to row block, so every scan result equals a
// first-true position on the scan's grid, found by binary search, one thread per row block:
//   asymmetric  start[i] = F(i), end[i] = max(F(i), E(i)) with
//               F(i) = first grid j with x1[i*bs] - x2[j] <= cutoff,
//               E(i) = first grid j with x2[j] - x1[last row of block i] > cutoff,
//               grid = {0, step, 2 step, ...} below n2, "none" = n2, step = align ? bs : 1;
//   symmetric   end[i] = first j in {bs, 2 bs, ...} below n with x[j] - x[last row] >= cutoff,
//               "none" = n (and end[0] = bs when bs >= n, as the scan never starts);
//               start[k] = bs * min{ i <= k : ceil(end[i] / bs) > k }, "none" = n, start[0] = 0.
#include "km_common.h"
#include "km_launch.h"

#include <algorithm>

namespace km {

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

void host_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1, int64_t n2,
                      float cutoff, int bs, bool align, int32_t* start, int32_t* end) {
    const int64_t rows = ceil_div(n1, bs);
    const int64_t step = align ? bs : 1;
    for (int64_t b = 0; b < num_batch; b++) {
        const float* a1 = x1 + b * n1;
        const float* a2 = x2 + b * n2;
        int32_t* s = start + b * rows;
        int32_t* e = end + b * rows;
        int64_t lo = 0;  // running start
        int64_t hi = 0;  // running end
        for (int64_t i = 0; i < rows; i++) {
            const float first = a1[i * bs];
            const float last = a1[std::min<int64_t>(i * bs + bs, n1) - 1];
            while (lo < n2) {
                const float tau = first - a2[lo];
                if (tau <= cutoff) break;
                lo = std::min<int64_t>(lo + step, n2);
            }
            s[i] = (int32_t)lo;
            hi = std::max(hi, lo);
            while (hi < n2) {
                const float tau = a2[hi] - last;
                if (tau > cutoff) break;
                hi = std::min<int64_t>(hi + step, n2);
            }
            e[i] = (int32_t)hi;
        }
    }
}

void host_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff, int bs,
                                int32_t* start, int32_t* end) {
    const int64_t rows = ceil_div(n, bs);
    for (int64_t b = 0; b < num_batch; b++) {
        const float* a = x + b * n;
        int32_t* s = start + b * rows;
        int32_t* e = end + b * rows;
        std::fill(s, s + rows, (int32_t)n);
        if (rows > 0) s[0] = 0;
        int64_t j = bs;
        for (int64_t i = 0; i < rows; i++) {
            const float last = a[std::min<int64_t>((i + 1) * bs, n) - 1];
            while (j < n) {
                const float tau = a[j] - last;
                if (tau >= cutoff) break;
                j = std::min<int64_t>(j + bs, n);
            }
            e[i] = (int32_t)j;
            const int64_t covered = ceil_div(j, bs);
            for (int64_t k = i; k < covered && k < rows; k++) {
                s[k] = std::min<int32_t>(s[k], (int32_t)(i * bs));
            }
        }
    }
}

void host_transpose_ranges(const int32_t* start, const int32_t* end, int64_t num_batch,
                           int64_t rows, int x1_size, int x2_size, int bs, int32_t* start_t,
                           int32_t* end_t) {
    const int64_t cols = ceil_div(x2_size, bs);
    for (int64_t b = 0; b < num_batch; b++) {
        const int32_t* s = start + b * rows;
        const int32_t* e = end + b * rows;
        int32_t* st = start_t + b * cols;
        int32_t* et = end_t + b * cols;
        std::fill(st, st + cols, (int32_t)x1_size);
        std::fill(et, et + cols, 0);
        for (int64_t i = 0; i < rows; i++) {
            if (s[i] == e[i]) continue;
            const int64_t cb0 = s[i] / bs;
            const int64_t cb1 = std::min<int64_t>(ceil_div(e[i], bs), cols);
            const int32_t r0 = (int32_t)(i * bs);
            const int32_t r1 = (int32_t)std::min<int64_t>(i * bs + bs, x1_size);
            for (int64_t j = cb0; j < cb1; j++) {
                st[j] = std::min(st[j], r0);
                et[j] = std::max(et[j], r1);
            }
        }
        // Column blocks no row touches become empty ranges that keep start monotone.
        if (cols > 0 && st[0] == x1_size) {
            st[0] = 0;
            et[0] = 0;
        }
        for (int64_t j = 1; j < cols; j++) {
            if (st[j] == x1_size) {
                st[j] = st[j - 1];
                et[j] = st[j - 1];
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Device versions.
// ---------------------------------------------------------------------------------------
struct RangeArgs {
    const float* x1;
    const float* x2;
    long long num_batch, n1, n2, rows;
    float cutoff;
    int bs;
    int step;
    int* start;
    int* end;
};

__global__ void __launch_bounds__(256) ranges_asym_kernel(const RangeArgs a) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= a.num_batch * a.rows) {
        return;
    }
    const long long b = t / a.rows;
    const long long i = t % a.rows;
    const float* __restrict__ x1 = a.x1 + b * a.n1;
    const float* __restrict__ x2 = a.x2 + b * a.n2;
    const float first = x1[i * a.bs];
    const float last = x1[min(i * a.bs + a.bs, a.n1) - 1];
    const long long grid = (a.n2 + a.step - 1) / a.step;

    // F: first grid point with first - x2[j] <= cutoff.
    long long lo = 0, hi = grid;
    while (lo < hi) {
        const long long mid = (lo + hi) >> 1;
        const float tau = first - x2[mid * a.step];
        if (tau <= a.cutoff) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    const long long f = min(lo * a.step, a.n2);

    // E: first grid point with x2[j] - last > cutoff.
    lo = 0;
    hi = grid;
    while (lo < hi) {
        const long long mid = (lo + hi) >> 1;
        const float tau = x2[mid * a.step] - last;
        if (tau > a.cutoff) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    const long long e = min(lo * a.step, a.n2);

    a.start[t] = (int)f;
    a.end[t] = (int)max(f, e);
}

__global__ void __launch_bounds__(256) ranges_sym_end_kernel(const RangeArgs a) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= a.num_batch * a.rows) {
        return;
    }
    const long long b = t / a.rows;
    const long long i = t % a.rows;
    const float* __restrict__ x = a.x1 + b * a.n1;
    const long long n = a.n1;
    if (a.bs >= n) {
        a.end[t] = a.bs;  // single row block; the scan never starts
        return;
    }
    const float last = x[min((i + 1) * a.bs, n) - 1];
    // Grid points g * bs for g in [1, grid), then n.
    const long long grid = (n + a.bs - 1) / a.bs;
    long long lo = 1, hi = grid;
    while (lo < hi) {
        const long long mid = (lo + hi) >> 1;
        const float tau = x[mid * a.bs] - last;
        if (tau >= a.cutoff) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    a.end[t] = (int)min(lo * a.bs, n);
}

__global__ void __launch_bounds__(256) ranges_sym_start_kernel(const RangeArgs a) {
    const long long t = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= a.num_batch * a.rows) {
        return;
    }
    const long long b = t / a.rows;
    const long long k = t % a.rows;
    const int* __restrict__ end = a.end + b * a.rows;
    // First i in [0, k] whose range reaches column block k.
    long long lo = 0, hi = k + 1;
    while (lo < hi) {
        const long long mid = (lo + hi) >> 1;
        const long long covered = ((long long)end[mid] + a.bs - 1) / a.bs;
        if (covered > k) {
            hi = mid;
        } else {
            lo = mid + 1;
        }
    }
    int value = lo <= k ? (int)(lo * a.bs) : (int)a.n1;
    if (k == 0) {
        value = 0;
    }
    a.start[t] = value;
}

hipError_t launch_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1,
                              int64_t n2, float cutoff, int block_size, int align, int32_t* start,
                              int32_t* end, hipStream_t stream) {
    RangeArgs a;
    a.x1 = x1;
    a.x2 = x2;
    a.num_batch = num_batch;
    a.n1 = n1;
    a.n2 = n2;
    a.rows = ceil_div(n1, block_size);
    a.cutoff = cutoff;
    a.bs = block_size;
    a.step = align ? block_size : 1;
    a.start = start;
    a.end = end;
    const long long total = a.num_batch * a.rows;
    if (total == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(ranges_asym_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0,
                       stream, a);
    return hipGetLastError();
}

hipError_t launch_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff,
                                        int block_size, int32_t* start, int32_t* end,
                                        hipStream_t stream) {
    RangeArgs a;
    a.x1 = x;
    a.x2 = x;
    a.num_batch = num_batch;
    a.n1 = n;
    a.n2 = n;
    a.rows = ceil_div(n, block_size);
    a.cutoff = cutoff;
    a.bs = block_size;
    a.step = block_size;
    a.start = start;
    a.end = end;
    const long long total = a.num_batch * a.rows;
    if (total == 0) {
        return hipSuccess;
    }
    const unsigned grid = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(ranges_sym_end_kernel, dim3(grid), dim3(256), 0, stream, a);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) {
        return err;
    }
    hipLaunchKernelGGL(ranges_sym_start_kernel, dim3(grid), dim3(256), 0, stream, a);
    return hipGetLastError();
}

}  // namespace km
