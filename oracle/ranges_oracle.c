/*
 * Range-builder oracle.  TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).
 *
 * Plain C restatement of the three functions of the reference's
 * native/ranges/ranges.cpp, statement by statement:
 *   oracle_make_ranges            ranges.cpp:8-62
 *   oracle_make_ranges_symmetric  ranges.cpp:64-101
 *   oracle_transpose_ranges       ranges.cpp:103-150
 * Arrays are contiguous [num_batch][len].  Every comparison is an fp32 subtraction followed
 * by an fp32 compare with the fp32 cutoff, as in the reference (float accessors, `const float
 * cutoff`).  Quirks are kept: with align the start scan only tests block-aligned columns; the
 * symmetric scan uses >= where the asymmetric one uses >; a symmetric pattern over fewer
 * points than one block reports end[0] = block_size.
 *
 * Pinned by tests/test_oracle_ranges.py: the reference's literal known answer
 * (tests/test_ranges.py:193-199), the property suite of tests/test_ranges.py:77-190, golden
 * vectors produced by the reference's own ranges.cpp compiled into oracle/_ref (committed
 * under tests/golden/), and a direct comparison with oracle/_ref when it is built.
 */
#include <stdint.h>

static int imin(int a, int b) { return a < b ? a : b; }
static int imax(int a, int b) { return a > b ? a : b; }
static int ceil_div(int a, int b) { return (a + b - 1) / b; }

void oracle_make_ranges(const float* x1, const float* x2, int num_batch, int n1, int n2,
                        float cutoff, int block_size, int align, int32_t* start, int32_t* end) {
    const int rows = ceil_div(n1, block_size);
    const int step = align ? block_size : 1;
    for (int batch = 0; batch < num_batch; batch++) {
        const float* x1_ = x1 + (int64_t)batch * n1;
        const float* x2_ = x2 + (int64_t)batch * n2;
        int32_t* start_ = start + (int64_t)batch * rows;
        int32_t* end_ = end + (int64_t)batch * rows;
        for (int i = 0; i < rows; i++) {
            const int row_first = i * block_size;
            int j = (i == 0) ? 0 : start_[i - 1];
            for (; j < n2; j = imin(j + step, n2)) {
                const float tau = x1_[row_first] - x2_[j];
                if (tau <= cutoff) {
                    break;
                }
            }
            start_[i] = j;

            const int row_last = imin(row_first + block_size, n1) - 1;
            j = (i == 0) ? 0 : end_[i - 1];
            if (j < start_[i]) {
                j = start_[i];
            }
            for (; j < n2; j = imin(j + step, n2)) {
                const float tau = x2_[j] - x1_[row_last];
                if (tau > cutoff) {
                    break;
                }
            }
            end_[i] = j;
        }
    }
}

void oracle_make_ranges_symmetric(const float* x, int num_batch, int n, float cutoff,
                                  int block_size, int32_t* start, int32_t* end) {
    const int rows = ceil_div(n, block_size);
    for (int batch = 0; batch < num_batch; batch++) {
        const float* x_ = x + (int64_t)batch * n;
        int32_t* start_ = start + (int64_t)batch * rows;
        int32_t* end_ = end + (int64_t)batch * rows;
        for (int i = 0; i < rows; i++) {
            start_[i] = n;
            end_[i] = 0;
        }
        if (rows > 0) {
            start_[0] = 0;
        }
        for (int i = 0; i < rows; i++) {
            const int row_last = imin((i + 1) * block_size, n) - 1;
            int j = (i == 0) ? block_size : end_[i - 1];
            for (; j < n; j = imin(j + block_size, n)) {
                const float tau = x_[j] - x_[row_last];
                if (tau >= cutoff) {
                    break;
                }
            }
            end_[i] = j;
            for (int k = i; k < ceil_div(j, block_size); k++) {
                start_[k] = imin(start_[k], i * block_size);
            }
        }
    }
}

void oracle_transpose_ranges(const int32_t* start, const int32_t* end, int num_batch, int rows,
                             int x1_size, int x2_size, int block_size, int32_t* start_t,
                             int32_t* end_t) {
    const int cols = ceil_div(x2_size, block_size);
    for (int batch = 0; batch < num_batch; batch++) {
        const int32_t* start_ = start + (int64_t)batch * rows;
        const int32_t* end_ = end + (int64_t)batch * rows;
        int32_t* start_t_ = start_t + (int64_t)batch * cols;
        int32_t* end_t_ = end_t + (int64_t)batch * cols;
        for (int j = 0; j < cols; j++) {
            start_t_[j] = x1_size;
            end_t_[j] = 0;
        }
        for (int i = 0; i < rows; i++) {
            if (start_[i] == end_[i]) {
                continue;
            }
            const int block_start = start_[i] / block_size;
            const int block_end = block_size == 1 ? end_[i] : ceil_div(end_[i], block_size);
            const int row_start = i * block_size;
            const int row_end = imin(row_start + block_size, x1_size);
            for (int j = block_start; j < block_end; j++) {
                start_t_[j] = imin(start_t_[j], row_start);
                end_t_[j] = imax(end_t_[j], row_end);
            }
        }
        if (cols > 0 && start_t_[0] == x1_size) {
            start_t_[0] = 0;
            end_t_[0] = 0;
        }
        for (int j = 1; j < cols; j++) {
            if (start_t_[j] == x1_size) {
                start_t_[j] = start_t_[j - 1];
                end_t_[j] = start_t_[j - 1];
            }
        }
    }
}
