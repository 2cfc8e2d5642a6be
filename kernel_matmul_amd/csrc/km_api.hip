// C-ABI entry points: argument validation, the gfx950 launch table, error reporting.
// Nothing here throws; every failure becomes a negative status plus a thread-local message.
#include "km_common.h"
#include "km_launch.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

namespace km {

void host_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1, int64_t n2,
                      float cutoff, int bs, bool align, int32_t* start, int32_t* end);
void host_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff, int bs,
                                int32_t* start, int32_t* end);
void host_transpose_ranges(const int32_t* start, const int32_t* end, int64_t num_batch,
                           int64_t rows, int x1_size, int x2_size, int bs, int32_t* start_t,
                           int32_t* end_t);

static thread_local char g_error[512] = "";

static int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return code;
}

static int fail_hip(const char* what, hipError_t err) {
    return fail(KM_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(err));
}

static const long long INT_LIMIT = 2147483647LL;

// Validates the shared part of every device entry point; returns the number of batch items
// through `num_batches` (0 is legal: nothing to do).
static int check_common(const char* op, int kernel_type, int batch_rank, const int64_t* batch_sizes,
                        int64_t m, int64_t n, long long* num_batches) {
    if (km_num_params(kernel_type) < 0) {
        return fail(KM_ERR_UNSUPPORTED, "%s: unknown kernel type %d", op, kernel_type);
    }
    if (batch_rank < 0 || batch_rank > KM_MAX_BATCH_RANK) {
        return fail(KM_ERR_UNSUPPORTED, "%s: batch rank %d outside [0, %d]", op, batch_rank,
                    KM_MAX_BATCH_RANK);
    }
    if (batch_rank > 0 && batch_sizes == nullptr) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: batch_sizes is NULL", op);
    }
    long long nb = 1;
    for (int d = 0; d < batch_rank; d++) {
        if (batch_sizes[d] < 0 || batch_sizes[d] > INT_LIMIT) {
            return fail(KM_ERR_INVALID_ARGUMENT, "%s: batch size %lld out of range", op,
                        (long long)batch_sizes[d]);
        }
        nb *= batch_sizes[d];
        if (nb > INT_LIMIT) {
            return fail(KM_ERR_UNSUPPORTED, "%s: more than 2^31-1 batch items", op);
        }
    }
    if (m < 0 || n < 0 || m > INT_LIMIT - KM_BLOCK_SIZE || n > INT_LIMIT - KM_BLOCK_SIZE) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: matrix size (%lld, %lld) out of range", op,
                    (long long)m, (long long)n);
    }
    *num_batches = nb;
    return KM_OK;
}

#define KM_REQUIRE_PTR(op, p)                                                     \
    do {                                                                          \
        if ((p) == nullptr) {                                                     \
            return fail(KM_ERR_INVALID_ARGUMENT, "%s: %s is NULL", (op), #p);    \
        }                                                                         \
    } while (0)

// ---------------------------------------------------------------------------------------
// gfx950 launch table for the forward operator.  256 CUs x 4 SIMDs: aim for at least one
// wavefront per SIMD.  Large problems run one wavefront per 128-row block (8 row groups,
// no cross-wavefront reduction); smaller ones first shrink the rows per wavefront, then
// let several wavefronts share a row range.  Fewer rows per wavefront repeat the rhs-operand
// work and shared row ranges add a reduction, so neither goes further than filling the SIMDs
// (measured: 1024 beats 2048 and 4096 from 157 to 3128 row-block items).
// ---------------------------------------------------------------------------------------
static const long long TARGET_WAVES = 1024;
// Row-block items from which the workgroup-shared forward kernel is considered.
static const long long BLOCK_VARIANT_MIN_ITEMS = 4096;

static int make_plan(const MatmulProblem& p, const km_launch_options* opt, MatmulPlan* plan) {
    int variant = opt ? opt->variant : KM_VARIANT_AUTO;
    plan->phase_split = 0;
    plan->group_tail = -1;
    plan->group_tail_halves = -1;
    if (opt && opt->reserved >= 2) {
        // measurements: grouped launch with this many split items per XCD (low 16 bits); bits
        // above: 0 = the usual share of them as two halves of 64 rows, else that count + 1
        plan->group_tail = (opt->reserved - 2) & 0xffff;
        plan->group_tail_halves = ((opt->reserved - 2) >> 16) - 1;
    }
    if (variant == KM_VARIANT_AUTO) {
        // Measured on gfx950 (n = 1e5, k = 16): for the locally periodic kernel with enough row
        // blocks to fill the device several times, sharing the rhs operand between four row
        // blocks wins (batch 8: 133 against 154 us; batch 2: 52 against 49 us, hence the
        // threshold); rbf and spectral kernels are faster through the column tables with one
        // wavefront per row block (rbf, batch 8: 77 against 86 us; batch 64: 494 against 578 us).
        const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
        const bool shared = p.kernel_type == KM_KERNEL_LOCALLY_PERIODIC && p.k <= 16 &&
                            row_blocks * p.num_batches >= BLOCK_VARIANT_MIN_ITEMS &&
                            !(opt && (opt->rows_per_wave != 0 || opt->col_splits > 1));
        variant = shared ? KM_VARIANT_BLOCK : KM_VARIANT_MFMA_F16;
    }
    if (variant != KM_VARIANT_VALU && variant != KM_VARIANT_MFMA_F32 && variant != KM_VARIANT_MFMA_F16 &&
        variant != KM_VARIANT_MFMA_F16_DIRECT && variant != KM_VARIANT_BLOCK && variant != KM_VARIANT_MFMA_F32_DIRECT) {
        return fail(KM_ERR_INVALID_ARGUMENT, "km_matmul: unknown variant %d", variant);
    }
    if (variant == KM_VARIANT_BLOCK) {
        if (opt && (opt->rows_per_wave != 0 || opt->col_splits > 1)) {
            return fail(KM_ERR_INVALID_ARGUMENT,
                        "km_matmul: the workgroup-shared variant has a fixed decomposition");
        }
        plan->variant = variant;
        plan->k_chunk = p.k <= 16 ? 16 : 32;
        plan->row_groups = 8;
        plan->col_splits = 1;
        plan->tail_balance = !(opt && opt->reserved == 1);
        plan->phase_split = p.kernel_type == KM_KERNEL_SPECTRAL && p.k <= 16;
        return KM_OK;
    }
    plan->variant = variant;
    if (variant == KM_VARIANT_VALU) {
        plan->k_chunk = p.k > 8 ? 16 : (p.k > 4 ? 8 : 4);
        plan->row_groups = 8;
        plan->col_splits = 1;
        plan->tail_balance = 0;
        return KM_OK;
    }
    // Table kernel (column tables in LDS, separable exponent): rbf and spectral kernels with up
    // to 16 rhs columns, the spectral one in phase-split form (two accumulator sets per rhs
    // column group); spectral kernels with 17 to 32 columns with the cosine per entry from
    // tabulated phases (n = 1e5, k = 32, batch 8: 156.6 against 162.8 us direct; n = 1e6: 1.24
    // against 1.29 ms; the rbf kernel gains nothing from its tables there, 112.9 against 108.7 us).
    // Everything else evaluates directly.
    // The fp32 contraction goes through the same tables for rbf and spectral kernels up to 32
    // columns (cos(A - B) per entry from tabulated cos B / sin B); otherwise directly as well.
    const bool rbf_or_spectral = p.kernel_type == KM_KERNEL_SPECTRAL || p.kernel_type == KM_KERNEL_RBF;
    const bool table = (variant == KM_VARIANT_MFMA_F16 &&
                        ((p.k <= 16 && rbf_or_spectral) || (p.k <= 32 && p.kernel_type == KM_KERNEL_SPECTRAL))) ||
                       (variant == KM_VARIANT_MFMA_F32 && p.k <= 32 && rbf_or_spectral);
    const bool phase_split = variant == KM_VARIANT_MFMA_F16 && table && p.kernel_type == KM_KERNEL_SPECTRAL && p.k <= 16;
    if (variant == KM_VARIANT_MFMA_F16 && !table) {
        variant = KM_VARIANT_MFMA_F16_DIRECT;
        plan->variant = variant;
    }
    if (variant == KM_VARIANT_MFMA_F32 && !table) {
        variant = KM_VARIANT_MFMA_F32_DIRECT;
        plan->variant = variant;
    }
    plan->k_chunk = p.k <= 16 ? 16 : ((p.k <= 32 || phase_split) ? 32 : 64);
    const int G = plan->k_chunk / 16;
    const long long row_blocks = (p.m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    const long long base = row_blocks * p.num_batches * ((p.k + plan->k_chunk - 1) / plan->k_chunk);

    int R = 8;
    if (opt && opt->rows_per_wave != 0) {
        const int rows = opt->rows_per_wave;
        if (rows != 16 && rows != 32 && rows != 64 && rows != 128) {
            return fail(KM_ERR_INVALID_ARGUMENT, "km_matmul: rows_per_wave must be 16, 32, 64 or 128");
        }
        R = rows / 16;
    } else {
        while (R > 1 && base * (8 / R) < TARGET_WAVES) {
            R /= 2;
        }
    }
    // Register budget of the split-fp16 kernels: their operand buffers and accumulators grow with
    // the number of rhs column groups, so wide rhs tiles get fewer row groups per wavefront (no
    // spills, at least two wavefronts per SIMD: G * R = 16 takes 191 to 250 VGPRs).  Measured:
    // 4 row groups instead of 2 at k = 64 save 25-28 % (n = 1e5, batch 8: 228 against 305 us),
    // 8 instead of 4 at k = 32 save 7-12 % (n = 1e6: 1.30 against 1.39 ms).
    if (variant == KM_VARIANT_MFMA_F16 || variant == KM_VARIANT_MFMA_F16_DIRECT) {
        const int groups = phase_split ? 2 * G : G;
        const int max_r = groups == 1 ? 8 : (groups == 2 ? 8 : (groups == 4 ? 4 : 2));
        if (R > max_r) {
            R = max_r;
        }
    }
    // Kernels at 2 wavefronts per SIMD (the direct kernel at G * R = 16) want 2048 wavefronts
    // before column ranges stop being shared (rbf, n = 65536, k = 64, batch 1: 45.4 us with two
    // wavefronts per row range against 52.9 us with one); the others 1024.
    const bool two_per_simd = (variant == KM_VARIANT_MFMA_F16_DIRECT && G * R >= 16) ||
                              (variant == KM_VARIANT_MFMA_F16 && table && G == 2);
    const long long wave_target = two_per_simd ? 2 * TARGET_WAVES : TARGET_WAVES;
    // Table kernel, 128-row items, at least 1.4 items per SIMD: the grouped launch below (one item
    // per wavefront, the remainder split by columns) rather than column shares for every item.
    // Measured (spectral, k = 16): n = 1e5, batch 2 (196 items per XCD) 32.9 against 37.5 us, batch 4
    // (391) 60.3 against 64.1 us; n = 20000, batch 12 (236) 42.3 against 51.0 us; batch 8 (157, below
    // the bound) 36.9 against 36.6 us.
    const long long per_xcd_128 = (row_blocks * p.num_batches + KM_NUM_XCD - 1) / KM_NUM_XCD;
    const bool grouped_128 = table && G == 1 && R == 8 && per_xcd_128 >= 128 + 48 &&
                             !(opt && (opt->col_splits != 0 || opt->reserved == 1));
    int S = 1;
    if (opt && opt->col_splits != 0) {
        S = opt->col_splits;
        if (S < 1 || S > 8) {
            return fail(KM_ERR_INVALID_ARGUMENT, "km_matmul: col_splits must be 1 to 8");
        }
    } else if (grouped_128) {
        S = 1;
    } else if (table && !two_per_simd) {
        // Table kernels: the share count that leaves the fullest SIMD the least work,
        // ceil(wavefronts / 1024) pieces of 1 / S of an item at 8 % of overhead per doubling
        // (n = 20000, batch 4: 1256 wavefronts of 64 rows leave 232 SIMDs with two of them, 31 us;
        // two shares each, three quarter-size pieces at most, 26 us; with 1564 wavefronts
        // (n = 50000, batch 2) two shares would make it four pieces: 33 against 28 us).
        const long long waves = base * (8 / R);
        double best = 0.0;
        for (int s = 1; s <= 8; s *= 2) {
            const long long pieces = (waves * s + TARGET_WAVES - 1) / TARGET_WAVES;
            double overhead = 1.0;
            for (int t = 1; t < s; t *= 2) {
                overhead *= 1.08;
            }
            const double cost = (double)pieces / s * overhead;
            if (s == 1 || cost < best * 0.97) {
                best = cost;
                S = s;
            }
            if (waves * s >= 4 * TARGET_WAVES) {
                break;
            }
        }
    } else {
        while (S < 8 && base * (8 / R) * S < wave_target) {
            S *= 2;
        }
    }
    // LDS per workgroup must stay within 64 KiB: the cross-wavefront reduction buffer takes
    // S * R * G KiB and the table kernel's tables 8.1 KiB per wavefront.
    while (S > 1 && S * (R * G + (table ? 9 : 0)) > 64) {
        S /= 2;
    }
    plan->row_groups = R;
    plan->col_splits = S;
    plan->tail_balance = !(opt && opt->reserved == 1);  // reserved = 1 switches it off (measurements)
    // Table kernel with one wavefront per 128-row item and enough items to run several rounds
    // per SIMD: grouped launch (workgroups of 4 wavefronts) whose last items are split by
    // columns.  Measured at n = 1e5, k = 16 (782 items per XCD at batch 8): 12-19 % of an XCD's
    // items split this way is best (112.7 us against 118.7 us with 16-row tail pieces; batch 64:
    // 751 against 773 us); more than a third of a round of wavefronts (128 items) gains nothing.
    if (table && G == 1 && R == 8 && S == 1 && plan->tail_balance && plan->group_tail < 0) {
        const long long per_xcd = (row_blocks * p.num_batches + KM_NUM_XCD - 1) / KM_NUM_XCD;
        if (per_xcd >= 128 + 48 && per_xcd < 2 * 128) {
            // one item per SIMD unsplit, everything beyond it split
            plan->group_tail = per_xcd - 128;
        }
        if (per_xcd >= 2 * 128) {
            plan->group_tail = per_xcd / 7 < 128 ? per_xcd / 7 : 128;
            if (variant == KM_VARIANT_MFMA_F32) {
                // Four wavefronts per SIMD instead of three: the last resident round (512 per XCD)
                // should consist of split pieces.  Measured at n = 1e5, k = 16, batch 8: 178 us
                // with 111 split items, 164.5 with 160 of which 80 in halves, 166-167 up to 256.
                plan->group_tail = per_xcd / 5 < 160 ? per_xcd / 5 : 160;
                if (plan->group_tail_halves < 0) {
                    plan->group_tail_halves = plan->group_tail / 2;
                }
            }
        }
    }
    // Mid-size problems through the table kernel in 64-row items (the launch table's choice when
    // 128-row items would not fill the SIMDs once): whole rounds of one item per SIMD go one item
    // per wavefront, the remainder of every XCD is split by columns and dispatched last.  Measured
    // (spectral, k = 16) against column shares for every item: n = 20000, batch 5 (197 items per
    // XCD) 26.0 against 32.6 us, batch 6 (236) 30.0 against 33.0 us; n = 50000, batch 2 (196) 24.4
    // against 26.0 us; n = 1e5, batch 1 (196) 23.6 against 25.0 us.  With few items beyond one per
    // SIMD the long wavefronts run alone and cannot hide their own latencies (n = 20000, batch 4:
    // 157 per XCD, 26.1 against 22.7 us), hence the lower bound on the remainder.
    const bool mid = variant == KM_VARIANT_MFMA_F16 && table && G == 1 && R == 4 && plan->tail_balance &&
                     !(opt && (opt->col_splits != 0 || opt->rows_per_wave != 0));
    if (mid && plan->group_tail < 0) {
        const long long per_xcd = (row_blocks * 2 * p.num_batches + KM_NUM_XCD - 1) / KM_NUM_XCD;
        if (per_xcd >= 128 + 48) {
            plan->group_tail = per_xcd % 128;
            S = 1;
            plan->col_splits = 1;
        }
    }
    if (plan->group_tail >= 0 && table && G == 1 && (R == 8 || (R == 4 && variant == KM_VARIANT_MFMA_F16)) &&
        !(opt && opt->col_splits != 0)) {
        S = 1;  // an explicit tail asks for the grouped launch
        plan->col_splits = 1;
    }
    if (!(table && G == 1 && S == 1 && (R == 8 || (R == 4 && variant == KM_VARIANT_MFMA_F16)))) {
        plan->group_tail = -1;
    }
    if (R == 4) {
        plan->group_tail_halves = 0;
    }
    // The very last of the split items also run as two halves of 64 rows (pieces of an eighth of
    // an item; they repeat the column-side work).
    if (plan->group_tail_halves < 0) {
        plan->group_tail_halves = plan->group_tail > 0 ? plan->group_tail / 4 : 0;
    }
    return KM_OK;
}

}  // namespace km

using namespace km;

extern "C" {

const char* km_last_error(void) { return g_error; }

int km_version(void) { return 100; }

int km_num_params(int kernel_type) {
    switch (kernel_type) {
        case KM_KERNEL_RBF: return 2;
        case KM_KERNEL_SPECTRAL: return 3;
        case KM_KERNEL_LOCALLY_PERIODIC: return 4;
        default: return -1;
    }
}

// ---------------------------------------------------------------------------------------
// Ranges (host).
// ---------------------------------------------------------------------------------------
static int check_ranges(const char* op, int64_t num_batch, int64_t n1, int64_t n2, int block_size) {
    if (block_size <= 0) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: block_size must be positive", op);
    }
    if (num_batch < 0 || n1 < 0 || n2 < 0 || n1 > INT_LIMIT - block_size || n2 > INT_LIMIT - block_size) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
    }
    return KM_OK;
}

int km_make_ranges(const float* x1, const float* x2, int64_t num_batch, int64_t n1, int64_t n2,
                   float cutoff, int block_size, int align, int32_t* start, int32_t* end) {
    const char* op = "km_make_ranges";
    if (int rc = check_ranges(op, num_batch, n1, n2, block_size)) return rc;
    if (num_batch == 0 || n1 == 0) return KM_OK;
    KM_REQUIRE_PTR(op, x1);
    if (n2 > 0) KM_REQUIRE_PTR(op, x2);
    KM_REQUIRE_PTR(op, start);
    KM_REQUIRE_PTR(op, end);
    host_make_ranges(x1, x2, num_batch, n1, n2, cutoff, block_size, align != 0, start, end);
    return KM_OK;
}

int km_make_ranges_symmetric(const float* x, int64_t num_batch, int64_t n, float cutoff,
                             int block_size, int32_t* start, int32_t* end) {
    const char* op = "km_make_ranges_symmetric";
    if (int rc = check_ranges(op, num_batch, n, n, block_size)) return rc;
    if (num_batch == 0 || n == 0) return KM_OK;
    KM_REQUIRE_PTR(op, x);
    KM_REQUIRE_PTR(op, start);
    KM_REQUIRE_PTR(op, end);
    host_make_ranges_symmetric(x, num_batch, n, cutoff, block_size, start, end);
    return KM_OK;
}

int km_transpose_ranges(const int32_t* start, const int32_t* end, int64_t num_batch, int64_t rows,
                        int x1_size, int x2_size, int block_size, int32_t* start_t, int32_t* end_t) {
    const char* op = "km_transpose_ranges";
    if (block_size <= 0) return fail(KM_ERR_INVALID_ARGUMENT, "%s: block_size must be positive", op);
    if (num_batch < 0 || rows < 0 || x1_size < 0 || x2_size < 0) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: sizes out of range", op);
    }
    if (rows != ((int64_t)x1_size + block_size - 1) / block_size) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: rows (%lld) does not match ceil(x1_size / block_size)",
                    op, (long long)rows);
    }
    if (num_batch == 0 || x2_size == 0) return KM_OK;
    if (rows > 0) {
        KM_REQUIRE_PTR(op, start);
        KM_REQUIRE_PTR(op, end);
    }
    KM_REQUIRE_PTR(op, start_t);
    KM_REQUIRE_PTR(op, end_t);
    host_transpose_ranges(start, end, num_batch, rows, x1_size, x2_size, block_size, start_t, end_t);
    return KM_OK;
}

// ---------------------------------------------------------------------------------------
// Ranges (device).
// ---------------------------------------------------------------------------------------
int km_make_ranges_device(const float* x1, const float* x2, int64_t num_batch, int64_t n1,
                          int64_t n2, float cutoff, int block_size, int align, int32_t* start,
                          int32_t* end, void* stream) {
    const char* op = "km_make_ranges_device";
    if (int rc = check_ranges(op, num_batch, n1, n2, block_size)) return rc;
    if (num_batch == 0 || n1 == 0) return KM_OK;
    KM_REQUIRE_PTR(op, x1);
    if (n2 > 0) KM_REQUIRE_PTR(op, x2);
    KM_REQUIRE_PTR(op, start);
    KM_REQUIRE_PTR(op, end);
    hipError_t err = launch_make_ranges(x1, x2, num_batch, n1, n2, cutoff, block_size, align, start,
                                        end, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

int km_make_ranges_symmetric_device(const float* x, int64_t num_batch, int64_t n, float cutoff,
                                    int block_size, int32_t* start, int32_t* end, void* stream) {
    const char* op = "km_make_ranges_symmetric_device";
    if (int rc = check_ranges(op, num_batch, n, n, block_size)) return rc;
    if (num_batch == 0 || n == 0) return KM_OK;
    KM_REQUIRE_PTR(op, x);
    KM_REQUIRE_PTR(op, start);
    KM_REQUIRE_PTR(op, end);
    hipError_t err = launch_make_ranges_symmetric(x, num_batch, n, cutoff, block_size, start, end,
                                                  (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

// ---------------------------------------------------------------------------------------
// matmul
// ---------------------------------------------------------------------------------------
int km_matmul(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
              int64_t k, const float* x1, const int64_t* x1_strides, const float* x2,
              const int64_t* x2_strides, const float* rhs, const int64_t* rhs_strides,
              const float* params, const int64_t* params_strides, const int32_t* start,
              const int64_t* start_strides, const int32_t* end, const int64_t* end_strides,
              float* out, const km_launch_options* options, void* stream) {
    const char* op = "km_matmul";
    long long nb = 0;
    if (int rc = check_common(op, kernel_type, batch_rank, batch_sizes, m, n, &nb)) return rc;
    if (k < 0 || k > INT_LIMIT) return fail(KM_ERR_INVALID_ARGUMENT, "%s: k out of range", op);
    if ((long long)m * k > INT_LIMIT * 64LL) {
        return fail(KM_ERR_UNSUPPORTED, "%s: m * k too large", op);
    }
    if (nb == 0 || m == 0 || k == 0) return KM_OK;
    KM_REQUIRE_PTR(op, x1);
    KM_REQUIRE_PTR(op, x1_strides);
    KM_REQUIRE_PTR(op, x2_strides);
    KM_REQUIRE_PTR(op, rhs_strides);
    KM_REQUIRE_PTR(op, params);
    KM_REQUIRE_PTR(op, params_strides);
    KM_REQUIRE_PTR(op, start);
    KM_REQUIRE_PTR(op, start_strides);
    KM_REQUIRE_PTR(op, end);
    KM_REQUIRE_PTR(op, end_strides);
    KM_REQUIRE_PTR(op, out);
    if (n > 0) {
        KM_REQUIRE_PTR(op, x2);
        KM_REQUIRE_PTR(op, rhs);
    }

    // The kernels address x2 / rhs as a 64-bit wave-uniform base plus 32-bit byte offsets that
    // span up to 60 rows and 63 columns of rhs: (60 + 63) * 4 * 2^22 stays below 2^32.
    {
        const int64_t x2_s = x2_strides[batch_rank];
        const int64_t r_s0 = rhs_strides[batch_rank];
        const int64_t r_s1 = rhs_strides[batch_rank + 1];
        if (x2_s < 0 || r_s0 < 0 || r_s1 < 0 || x1_strides[batch_rank] < 0) {
            return fail(KM_ERR_UNSUPPORTED, "%s: negative strides are not supported", op);
        }
        if (x2_s > (1 << 22) || r_s0 > (1 << 22) || r_s1 > (1 << 22)) {
            return fail(KM_ERR_UNSUPPORTED, "%s: inner strides above 2^22 elements are not supported", op);
        }
    }

    MatmulProblem p;
    p.kernel_type = kernel_type;
    p.batch_rank = batch_rank;
    p.batch_sizes = batch_sizes;
    p.num_batches = nb;
    p.m = m;
    p.n = n;
    p.k = k;
    p.x1 = x1;
    p.x1_strides = x1_strides;
    p.x2 = x2;
    p.x2_strides = x2_strides;
    p.rhs = rhs;
    p.rhs_strides = rhs_strides;
    p.params = params;
    p.params_strides = params_strides;
    p.start = start;
    p.start_strides = start_strides;
    p.end = end;
    p.end_strides = end_strides;
    p.out = out;

    MatmulPlan plan;
    if (int rc = make_plan(p, options, &plan)) return rc;
    hipError_t err = launch_matmul(p, plan, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

int km_param_grad_describe(int kernel_type, int64_t num_batches, int64_t m, int64_t c, char* text,
                           size_t text_bytes) {
    const char* op = "km_param_grad_describe";
    if (km_num_params(kernel_type) < 0) {
        return fail(KM_ERR_UNSUPPORTED, "%s: unknown kernel type %d", op, kernel_type);
    }
    if (num_batches < 0 || m < 0 || c < 0 || text == nullptr || text_bytes == 0) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: invalid argument", op);
    }
    describe_param_grad(kernel_type, m, num_batches, c, text, text_bytes);
    return KM_OK;
}

int km_matmul_describe(int kernel_type, int64_t num_batches, int64_t m, int64_t n, int64_t k,
                       const km_launch_options* options, char* text, size_t text_bytes) {
    const char* op = "km_matmul_describe";
    if (km_num_params(kernel_type) < 0) {
        return fail(KM_ERR_UNSUPPORTED, "%s: unknown kernel type %d", op, kernel_type);
    }
    if (num_batches < 0 || m < 0 || n < 0 || k < 0 || text == nullptr || text_bytes == 0) {
        return fail(KM_ERR_INVALID_ARGUMENT, "%s: invalid argument", op);
    }
    MatmulProblem p;
    memset(&p, 0, sizeof(p));
    p.kernel_type = kernel_type;
    p.num_batches = num_batches;
    p.m = m;
    p.n = n;
    p.k = k;
    MatmulPlan plan;
    if (int rc = make_plan(p, options, &plan)) return rc;
    static const char* const kernels[] = {"rbf", "spectral", "locally_periodic"};
    const char* kt = kernels[kernel_type];
    const long long row_blocks = (m + KM_BLOCK_SIZE - 1) / KM_BLOCK_SIZE;
    const int G = plan.k_chunk / 16;
    switch (plan.variant) {
        case KM_VARIANT_VALU:
            snprintf(text, text_bytes, "km::fwd_valu<%s, KC=%d>: 128 rows per workgroup, %lld workgroups", kt,
                     plan.k_chunk, row_blocks * num_batches * ((k + plan.k_chunk - 1) / plan.k_chunk));
            break;
        case KM_VARIANT_BLOCK:
            snprintf(text, text_bytes,
                     "km::fwd_block<%s, phase_split=%d, G=%d>: 4 wavefronts per 4 row blocks, rhs operand shared in LDS",
                     kt, plan.phase_split, G);
            break;
        default: {
            const char* name = plan.variant == KM_VARIANT_MFMA_F32_DIRECT
                                   ? "km::fwd_mfma_f32"
                                   : (plan.variant == KM_VARIANT_MFMA_F32
                                          ? "km::fwd_table_f32"
                                          : (plan.variant == KM_VARIANT_MFMA_F16 ? "km::fwd_table_f16" : "km::fwd_mfma_f16"));
            if (plan.variant == KM_VARIANT_MFMA_F16 && plan.group_tail >= 0 && plan.row_groups == 4) {
                snprintf(text, text_bytes,
                         "%s_grouped64<%s>: 64 rows per wavefront, 4 wavefronts per workgroup, the last %lld "
                         "items of each XCD split by columns over a workgroup",
                         name, kt, plan.group_tail);
                break;
            }
            if ((plan.variant == KM_VARIANT_MFMA_F16 || plan.variant == KM_VARIANT_MFMA_F32) && plan.group_tail >= 0) {
                snprintf(text, text_bytes,
                         "%s_grouped<%s>: 128 rows per wavefront, 4 wavefronts per workgroup, the "
                         "last %lld items of each XCD split by columns over a workgroup (the last %lld of them "
                         "also into two halves of 64 rows)",
                         name, kt, plan.group_tail, plan.group_tail_halves);
                break;
            }
            snprintf(text, text_bytes, "%s<%s, G=%d, R=%d>: %d rows per wavefront, %d wavefront(s) per row range%s",
                     name, kt, G, plan.row_groups, 16 * plan.row_groups, plan.col_splits,
                     plan.tail_balance && plan.row_groups == 8 && plan.col_splits == 1 &&
                             plan.variant == KM_VARIANT_MFMA_F16_DIRECT &&
                             row_blocks * num_batches >= 2 * 128 * KM_NUM_XCD
                         ? ", tail items cut into 16-row pieces"
                         : "");
            break;
        }
    }
    return KM_OK;
}

// ---------------------------------------------------------------------------------------
// param_grad (matmul_bwd and bilinear_derivative)
// ---------------------------------------------------------------------------------------
size_t km_param_grad_workspace_size(int kernel_type, int batch_rank, const int64_t* batch_sizes,
                                    int64_t m, int64_t n, int64_t c) {
    long long nb = 0;
    if (check_common("km_param_grad_workspace_size", kernel_type, batch_rank, batch_sizes, m, n, &nb)) {
        return 0;
    }
    if (nb == 0 || m == 0) return 0;
    // Enough for either form of the first pass (which one runs also depends on the strides).
    long long rows = param_grad_partials_per_batch(m, nb);
    const long long feature_rows = param_grad_feature_partials_per_batch(kernel_type, m, nb, c);
    if (feature_rows > rows) rows = feature_rows;
    return (size_t)nb * (size_t)rows * KM_MAX_PARAMS * sizeof(float);
}

// Device scratch of the allocation-free entry point: one array per GPU, held until the
// process ends.  In host code the array's name is only a handle for hipGetSymbolAddress; the
// address each device keeps it at is looked up once per device and used from then on.
static __device__ __attribute__((used)) __align__(256) unsigned char scratch[KM_STATIC_SCRATCH_BYTES];

#define KM_MAX_DEVICES 64
static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[KM_MAX_DEVICES];  // per device, null until the first call there

// Address of `scratch` on the current device (looked up on the first call per device).
static int static_scratch(const char* op, void** ptr) {
    int device = -1;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return fail_hip(op, err);
    if (device < 0 || device >= KM_MAX_DEVICES) {
        return fail(KM_ERR_UNSUPPORTED, "%s: device ordinal %d not supported", op, device);
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device] == nullptr) {
        void* p = nullptr;
        err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (err != hipSuccess || p == nullptr) {
            return fail_hip(op, err != hipSuccess ? err : hipErrorInvalidSymbol);
        }
        g_scratch_ptr[device] = p;
    }
    *ptr = g_scratch_ptr[device];
    return KM_OK;
}

// Shared body of km_param_grad (caller's workspace) and km_param_grad_static (the library's
// per-device static scratch).
static int param_grad_entry(const char* op, bool use_static, int kernel_type, int batch_rank,
                            const int64_t* batch_sizes, int64_t m, int64_t n, int64_t c,
                            const float* x1, const int64_t* x1_strides, const float* x2,
                            const int64_t* x2_strides, const float* left,
                            const int64_t* left_strides, const float* right,
                            const int64_t* right_strides, const float* params,
                            const int64_t* params_strides, const int32_t* start,
                            const int64_t* start_strides, const int32_t* end,
                            const int64_t* end_strides, float* grad, void* workspace,
                            size_t workspace_bytes, void* stream) {
    long long nb = 0;
    if (int rc = check_common(op, kernel_type, batch_rank, batch_sizes, m, n, &nb)) return rc;
    if (c < 0 || c > INT_LIMIT) return fail(KM_ERR_INVALID_ARGUMENT, "%s: c out of range", op);
    if (nb == 0) return KM_OK;
    const size_t need = km_param_grad_workspace_size(kernel_type, batch_rank, batch_sizes, m, n, c);
    if (use_static && need > (size_t)KM_STATIC_SCRATCH_BYTES) {
        return fail(KM_ERR_WORKSPACE,
                    "%s: this problem needs %zu bytes of scratch, the static buffer holds %zu "
                    "(use km_param_grad with a caller-provided workspace)",
                    op, need, (size_t)KM_STATIC_SCRATCH_BYTES);
    }
    KM_REQUIRE_PTR(op, grad);
    KM_REQUIRE_PTR(op, params);
    KM_REQUIRE_PTR(op, params_strides);
    KM_REQUIRE_PTR(op, x1_strides);
    KM_REQUIRE_PTR(op, x2_strides);
    KM_REQUIRE_PTR(op, left_strides);
    KM_REQUIRE_PTR(op, right_strides);
    KM_REQUIRE_PTR(op, start_strides);
    KM_REQUIRE_PTR(op, end_strides);
    if (m > 0) {
        KM_REQUIRE_PTR(op, x1);
        KM_REQUIRE_PTR(op, start);
        KM_REQUIRE_PTR(op, end);
        if (c > 0) KM_REQUIRE_PTR(op, left);
    }
    if (n > 0) {
        KM_REQUIRE_PTR(op, x2);
        if (c > 0) KM_REQUIRE_PTR(op, right);
    }
    if (use_static) {
        if (int rc = static_scratch(op, &workspace)) return rc;
    } else if (need > 0 && (workspace == nullptr || workspace_bytes < need)) {
        return fail(KM_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", op, need,
                    workspace ? workspace_bytes : (size_t)0);
    }

    ParamGradProblem p;
    p.kernel_type = kernel_type;
    p.batch_rank = batch_rank;
    p.batch_sizes = batch_sizes;
    p.num_batches = nb;
    p.m = m;
    p.n = n;
    p.c = c;
    p.x1 = x1;
    p.x1_strides = x1_strides;
    p.x2 = x2;
    p.x2_strides = x2_strides;
    p.left = left;
    p.left_strides = left_strides;
    p.right = right;
    p.right_strides = right_strides;
    p.params = params;
    p.params_strides = params_strides;
    p.start = start;
    p.start_strides = start_strides;
    p.end = end;
    p.end_strides = end_strides;
    p.grad = grad;
    p.workspace = workspace;
    hipError_t err = launch_param_grad(p, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

int km_param_grad(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m,
                  int64_t n, int64_t c, const float* x1, const int64_t* x1_strides,
                  const float* x2, const int64_t* x2_strides, const float* left,
                  const int64_t* left_strides, const float* right, const int64_t* right_strides,
                  const float* params, const int64_t* params_strides, const int32_t* start,
                  const int64_t* start_strides, const int32_t* end, const int64_t* end_strides,
                  float* grad, void* workspace, size_t workspace_bytes, void* stream) {
    return param_grad_entry("km_param_grad", false, kernel_type, batch_rank, batch_sizes, m, n, c,
                            x1, x1_strides, x2, x2_strides, left, left_strides, right,
                            right_strides, params, params_strides, start, start_strides, end,
                            end_strides, grad, workspace, workspace_bytes, stream);
}

int km_param_grad_static(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m,
                         int64_t n, int64_t c, const float* x1, const int64_t* x1_strides,
                         const float* x2, const int64_t* x2_strides, const float* left,
                         const int64_t* left_strides, const float* right,
                         const int64_t* right_strides, const float* params,
                         const int64_t* params_strides, const int32_t* start,
                         const int64_t* start_strides, const int32_t* end,
                         const int64_t* end_strides, float* grad, void* stream) {
    return param_grad_entry("km_param_grad_static", true, kernel_type, batch_rank, batch_sizes, m, n,
                            c, x1, x1_strides, x2, x2_strides, left, left_strides, right,
                            right_strides, params, params_strides, start, start_strides, end,
                            end_strides, grad, nullptr, 0, stream);
}

// ---------------------------------------------------------------------------------------
// index
// ---------------------------------------------------------------------------------------
int km_index(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
             const float* x1, const int64_t* x1_strides, const float* x2,
             const int64_t* x2_strides, const float* params, const int64_t* params_strides,
             const int32_t* start, const int64_t* start_strides, const int32_t* end,
             const int64_t* end_strides, int index_rank, const int64_t* index_sizes,
             const int32_t* const* batch_index, const int64_t* const* batch_index_strides,
             const int32_t* row_index, const int64_t* row_index_strides,
             const int32_t* col_index, const int64_t* col_index_strides, float* out,
             void* stream) {
    const char* op = "km_index";
    long long nb = 0;
    if (int rc = check_common(op, kernel_type, batch_rank, batch_sizes, m, n, &nb)) return rc;
    if (index_rank < 1 || index_rank > KM_MAX_BATCH_RANK + 1) {
        return fail(KM_ERR_UNSUPPORTED, "%s: index rank %d outside [1, %d]", op, index_rank,
                    KM_MAX_BATCH_RANK + 1);
    }
    KM_REQUIRE_PTR(op, index_sizes);
    long long total = 1;
    for (int d = 0; d < index_rank; d++) {
        if (index_sizes[d] < 0) return fail(KM_ERR_INVALID_ARGUMENT, "%s: negative index size", op);
        total *= index_sizes[d];
        if (total > INT_LIMIT * 256LL) return fail(KM_ERR_UNSUPPORTED, "%s: too many index entries", op);
    }
    if (total == 0) return KM_OK;
    KM_REQUIRE_PTR(op, out);
    KM_REQUIRE_PTR(op, row_index);
    KM_REQUIRE_PTR(op, row_index_strides);
    KM_REQUIRE_PTR(op, col_index);
    KM_REQUIRE_PTR(op, col_index_strides);
    KM_REQUIRE_PTR(op, x1_strides);
    KM_REQUIRE_PTR(op, x2_strides);
    KM_REQUIRE_PTR(op, params_strides);
    KM_REQUIRE_PTR(op, start_strides);
    KM_REQUIRE_PTR(op, end_strides);
    if (batch_rank > 0) {
        KM_REQUIRE_PTR(op, batch_index);
        KM_REQUIRE_PTR(op, batch_index_strides);
        for (int d = 0; d < batch_rank; d++) {
            if (batch_index[d] == nullptr || batch_index_strides[d] == nullptr) {
                return fail(KM_ERR_INVALID_ARGUMENT, "%s: batch_index[%d] is NULL", op, d);
            }
        }
    }
    // With an empty matrix no entry can be inside it; the kernel then only writes zeros and
    // never dereferences the matrix inputs.
    const bool empty = nb == 0 || m == 0 || n == 0;
    if (!empty) {
        KM_REQUIRE_PTR(op, x1);
        KM_REQUIRE_PTR(op, x2);
        KM_REQUIRE_PTR(op, params);
        KM_REQUIRE_PTR(op, start);
        KM_REQUIRE_PTR(op, end);
    }

    IndexProblem p;
    p.kernel_type = kernel_type;
    p.batch_rank = batch_rank;
    p.batch_sizes = batch_sizes;
    p.m = empty ? 0 : m;
    p.n = empty ? 0 : n;
    p.x1 = x1;
    p.x1_strides = x1_strides;
    p.x2 = x2;
    p.x2_strides = x2_strides;
    p.params = params;
    p.params_strides = params_strides;
    p.start = start;
    p.start_strides = start_strides;
    p.end = end;
    p.end_strides = end_strides;
    p.index_rank = index_rank;
    p.index_sizes = index_sizes;
    p.batch_index = batch_index;
    p.batch_index_strides = batch_index_strides;
    p.row_index = row_index;
    p.row_index_strides = row_index_strides;
    p.col_index = col_index;
    p.col_index_strides = col_index_strides;
    p.out = out;
    hipError_t err = launch_index(p, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}


// ---------------------------------------------------------------------------------------
// index_bwd
// ---------------------------------------------------------------------------------------
size_t km_index_bwd_workspace_size(int64_t num_entries) {
    return num_entries > 0 ? index_bwd_workspace_bytes(num_entries) : 0;
}

int km_index_bwd(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
                 const float* x1, const int64_t* x1_strides, const float* x2,
                 const int64_t* x2_strides, const float* params, const int64_t* params_strides,
                 const int32_t* start, const int64_t* start_strides, const int32_t* end,
                 const int64_t* end_strides, int index_rank, const int64_t* index_sizes,
                 const int32_t* const* batch_index, const int64_t* const* batch_index_strides,
                 const int32_t* row_index, const int64_t* row_index_strides,
                 const int32_t* col_index, const int64_t* col_index_strides,
                 const float* out_grad, const int64_t* out_grad_strides, float* grad,
                 void* workspace, size_t workspace_bytes, void* stream) {
    const char* op = "km_index_bwd";
    long long nb = 0;
    if (int rc = check_common(op, kernel_type, batch_rank, batch_sizes, m, n, &nb)) return rc;
    if (index_rank < 1 || index_rank > KM_MAX_BATCH_RANK + 1) {
        return fail(KM_ERR_UNSUPPORTED, "%s: index rank %d outside [1, %d]", op, index_rank,
                    KM_MAX_BATCH_RANK + 1);
    }
    KM_REQUIRE_PTR(op, index_sizes);
    long long total = 1;
    for (int d = 0; d < index_rank; d++) {
        if (index_sizes[d] < 0) return fail(KM_ERR_INVALID_ARGUMENT, "%s: negative index size", op);
        total *= index_sizes[d];
        if (total > INT_LIMIT) return fail(KM_ERR_UNSUPPORTED, "%s: too many index entries", op);
    }
    if (nb == 0) return KM_OK;
    KM_REQUIRE_PTR(op, grad);
    KM_REQUIRE_PTR(op, params);
    KM_REQUIRE_PTR(op, params_strides);
    KM_REQUIRE_PTR(op, x1_strides);
    KM_REQUIRE_PTR(op, x2_strides);
    KM_REQUIRE_PTR(op, start_strides);
    KM_REQUIRE_PTR(op, end_strides);
    if (total > 0) {
        KM_REQUIRE_PTR(op, row_index);
        KM_REQUIRE_PTR(op, row_index_strides);
        KM_REQUIRE_PTR(op, col_index);
        KM_REQUIRE_PTR(op, col_index_strides);
        KM_REQUIRE_PTR(op, out_grad);
        KM_REQUIRE_PTR(op, out_grad_strides);
        if (batch_rank > 0) {
            KM_REQUIRE_PTR(op, batch_index);
            KM_REQUIRE_PTR(op, batch_index_strides);
            for (int d = 0; d < batch_rank; d++) {
                if (batch_index[d] == nullptr || batch_index_strides[d] == nullptr) {
                    return fail(KM_ERR_INVALID_ARGUMENT, "%s: batch_index[%d] is NULL", op, d);
                }
            }
        }
    }
    const bool empty = m == 0 || n == 0;
    if (!empty && total > 0) {
        KM_REQUIRE_PTR(op, x1);
        KM_REQUIRE_PTR(op, x2);
        KM_REQUIRE_PTR(op, start);
        KM_REQUIRE_PTR(op, end);
    }
    const size_t need = km_index_bwd_workspace_size(total);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need)) {
        return fail(KM_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", op, need,
                    workspace ? workspace_bytes : (size_t)0);
    }
    IndexBwdProblem p;
    p.index.kernel_type = kernel_type;
    p.index.batch_rank = batch_rank;
    p.index.batch_sizes = batch_sizes;
    p.index.m = empty ? 0 : m;
    p.index.n = empty ? 0 : n;
    p.index.x1 = x1;
    p.index.x1_strides = x1_strides;
    p.index.x2 = x2;
    p.index.x2_strides = x2_strides;
    p.index.params = params;
    p.index.params_strides = params_strides;
    p.index.start = start;
    p.index.start_strides = start_strides;
    p.index.end = end;
    p.index.end_strides = end_strides;
    p.index.index_rank = index_rank;
    p.index.index_sizes = index_sizes;
    p.index.batch_index = batch_index;
    p.index.batch_index_strides = batch_index_strides;
    p.index.row_index = row_index;
    p.index.row_index_strides = row_index_strides;
    p.index.col_index = col_index;
    p.index.col_index_strides = col_index_strides;
    p.index.out = nullptr;
    p.num_batches = nb;
    p.out_grad = out_grad;
    p.out_grad_strides = out_grad_strides;
    p.grad = grad;
    p.workspace = workspace;
    hipError_t err = launch_index_bwd(p, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

// ---------------------------------------------------------------------------------------
// dense / dense_bwd
// ---------------------------------------------------------------------------------------
static int fill_dense(const char* op, DenseProblem* p, int kernel_type, int batch_rank,
                      const int64_t* batch_sizes, int64_t m, int64_t n, const float* x1,
                      const int64_t* x1_strides, const float* x2, const int64_t* x2_strides,
                      const float* params, const int64_t* params_strides, const int32_t* start,
                      const int64_t* start_strides, const int32_t* end, const int64_t* end_strides,
                      long long* nb) {
    if (int rc = check_common(op, kernel_type, batch_rank, batch_sizes, m, n, nb)) return rc;
    if (*nb == 0) return KM_OK;
    KM_REQUIRE_PTR(op, params);
    KM_REQUIRE_PTR(op, params_strides);
    KM_REQUIRE_PTR(op, x1_strides);
    KM_REQUIRE_PTR(op, x2_strides);
    KM_REQUIRE_PTR(op, start_strides);
    KM_REQUIRE_PTR(op, end_strides);
    if (m > 0) {
        KM_REQUIRE_PTR(op, x1);
        KM_REQUIRE_PTR(op, start);
        KM_REQUIRE_PTR(op, end);
    }
    if (n > 0) KM_REQUIRE_PTR(op, x2);
    p->kernel_type = kernel_type;
    p->batch_rank = batch_rank;
    p->batch_sizes = batch_sizes;
    p->num_batches = *nb;
    p->m = m;
    p->n = n;
    p->x1 = x1;
    p->x1_strides = x1_strides;
    p->x2 = x2;
    p->x2_strides = x2_strides;
    p->params = params;
    p->params_strides = params_strides;
    p->start = start;
    p->start_strides = start_strides;
    p->end = end;
    p->end_strides = end_strides;
    p->out = nullptr;
    p->weights = nullptr;
    p->weights_strides = nullptr;
    p->grad = nullptr;
    p->workspace = nullptr;
    return KM_OK;
}

int km_dense(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
             const float* x1, const int64_t* x1_strides, const float* x2,
             const int64_t* x2_strides, const float* params, const int64_t* params_strides,
             const int32_t* start, const int64_t* start_strides, const int32_t* end,
             const int64_t* end_strides, float* out, void* stream) {
    const char* op = "km_dense";
    DenseProblem p;
    long long nb = 0;
    if (int rc = fill_dense(op, &p, kernel_type, batch_rank, batch_sizes, m, n, x1, x1_strides, x2,
                            x2_strides, params, params_strides, start, start_strides, end,
                            end_strides, &nb)) {
        return rc;
    }
    if (nb == 0 || m == 0 || n == 0) return KM_OK;
    KM_REQUIRE_PTR(op, out);
    p.out = out;
    hipError_t err = launch_dense(p, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

int km_dense_bwd(int kernel_type, int batch_rank, const int64_t* batch_sizes, int64_t m, int64_t n,
                 const float* x1, const int64_t* x1_strides, const float* x2,
                 const int64_t* x2_strides, const float* params, const int64_t* params_strides,
                 const int32_t* start, const int64_t* start_strides, const int32_t* end,
                 const int64_t* end_strides, const float* out_grad,
                 const int64_t* out_grad_strides, float* grad, void* workspace,
                 size_t workspace_bytes, void* stream) {
    const char* op = "km_dense_bwd";
    DenseProblem p;
    long long nb = 0;
    if (int rc = fill_dense(op, &p, kernel_type, batch_rank, batch_sizes, m, n, x1, x1_strides, x2,
                            x2_strides, params, params_strides, start, start_strides, end,
                            end_strides, &nb)) {
        return rc;
    }
    if (nb == 0) return KM_OK;
    KM_REQUIRE_PTR(op, grad);
    KM_REQUIRE_PTR(op, out_grad_strides);
    if (m > 0 && n > 0) KM_REQUIRE_PTR(op, out_grad);
    const size_t need = km_param_grad_workspace_size(kernel_type, batch_rank, batch_sizes, m, n, 0);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need)) {
        return fail(KM_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", op, need,
                    workspace ? workspace_bytes : (size_t)0);
    }
    p.weights = out_grad;
    p.weights_strides = out_grad_strides;
    p.grad = grad;
    p.workspace = workspace;
    hipError_t err = launch_dense_bwd(p, (hipStream_t)stream);
    return err == hipSuccess ? KM_OK : fail_hip(op, err);
}

}  // extern "C"
