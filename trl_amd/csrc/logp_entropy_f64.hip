// fp64 logits: the log-prob / entropy forward and its backward in double precision.
//
// The reference treats float64 like float32 (`logsumexp` branch of selective_log_softmax, trl/trainer/utils.py:506-510;
// its unit test runs both, tests/test_utils.py:866-905).  Nothing trains on fp64 logits, so these kernels are written
// for exactness, not bandwidth: one workgroup per row, two sweeps in the forward (row maximum, then the sums relative
// to it), libm `exp` / `log`, double accumulators combined in a fixed order.
#include "common.hpp"

namespace trlk {
namespace {

constexpr int kT64 = 256;

__device__ __forceinline__ double wave_sum_f64(double v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ double wave_max_f64(double v) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) v = fmax(v, __shfl_xor(v, o));
    return v;
}

struct Fwd64 {
    const double* logits;
    int64_t rows_per_seq, vocab, seq_stride, row_stride;
    const int64_t* index;
    int32_t n_index;
    double inv_t;
    const uint8_t* row_mask;
    double *out_logp, *out_entropy, *out_lse;
    int32_t* error_flag;
};

__global__ __launch_bounds__(kT64) void logp_entropy_fwd_f64_kernel(Fwd64 a) {
    __shared__ double red[2][kT64 / kWave];
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int64_t row = blockIdx.x;
    const int64_t b = row / a.rows_per_seq, t = row - b * a.rows_per_seq;
    if (a.row_mask && a.row_mask[row] == 0) {  // skipped row: outputs 0, nothing read
        if (tid == 0) {
            if (a.out_entropy) a.out_entropy[row] = 0.0;
            if (a.out_lse) a.out_lse[row] = 0.0;
        }
        for (int k = tid; k < a.n_index; k += kT64) a.out_logp[row * a.n_index + k] = 0.0;
        return;
    }
    const double* x = a.logits + b * a.seq_stride + t * a.row_stride;
    double m = -INFINITY;
    for (int64_t v = tid; v < a.vocab; v += kT64) m = fmax(m, x[v]);
    m = wave_max_f64(m);
    if (lane == 0) red[0][wave] = m;
    __syncthreads();
    double M = red[0][0];
    for (int w = 1; w < kT64 / kWave; ++w) M = fmax(M, red[0][w]);
    __syncthreads();
    double s = 0.0, u = 0.0;
    for (int64_t v = tid; v < a.vocab; v += kT64) {
        const double e = exp((x[v] - M) * a.inv_t);
        s += e;
        u += e * x[v];
    }
    s = wave_sum_f64(s);
    u = wave_sum_f64(u);
    if (lane == 0) {
        red[0][wave] = s;
        red[1][wave] = u;
    }
    __syncthreads();
    double S = 0.0, U = 0.0;
    for (int w = 0; w < kT64 / kWave; ++w) {
        S += red[0][w];
        U += red[1][w];
    }
    const double lse = M * a.inv_t + log(S);
    if (tid == 0) {
        if (a.out_entropy) a.out_entropy[row] = lse - (U / S) * a.inv_t;
        if (a.out_lse) a.out_lse[row] = lse;
    }
    for (int k = tid; k < a.n_index; k += kT64) {
        const int64_t idx = a.index[row * a.n_index + k];
        if (idx >= 0 && idx < a.vocab) {
            a.out_logp[row * a.n_index + k] = x[idx] * a.inv_t - lse;
        } else {
            a.out_logp[row * a.n_index + k] = NAN;
            if (a.error_flag) atomicOr(a.error_flag, TRLK_FLAG_INDEX_OUT_OF_RANGE);
        }
    }
}

struct Bwd64 {
    const double* logits;
    int64_t rows_per_seq, vocab, seq_stride, row_stride;
    const int64_t* index;
    int32_t n_index;
    double inv_t;
    const double *lse, *entropy, *g_logp, *g_entropy;
    double* dlogits;
    int64_t out_rows_per_seq, out_row_offset, out_seq_stride, out_row_stride;
};

// dlogits[v] = p_v * (-(sum_k g_k) - h * ((z_v - lse) + H)) / T  (+ g_k / T at v = index[k]),  z = x / T
__global__ __launch_bounds__(kT64) void logp_entropy_bwd_f64_kernel(Bwd64 a) {
    const int tid = threadIdx.x;
    const int64_t orow = blockIdx.x;
    const int64_t b = orow / a.out_rows_per_seq, to = orow - b * a.out_rows_per_seq, t = to - a.out_row_offset;
    double* out = a.dlogits + b * a.out_seq_stride + to * a.out_row_stride;
    bool live = t >= 0 && t < a.rows_per_seq;
    const int64_t row = b * a.rows_per_seq + (live ? t : 0);
    double gsum = 0.0;
    bool any = false;
    if (live)
        for (int k = 0; k < a.n_index; ++k) {
            const double g = a.g_logp[row * a.n_index + k];
            gsum += g;
            any |= g != 0.0;
        }
    const double h = (live && a.g_entropy) ? a.g_entropy[row] : 0.0;
    live = live && (any || h != 0.0);
    if (!live) {
        for (int64_t v = tid; v < a.vocab; v += kT64) out[v] = 0.0;
        return;
    }
    const double* x = a.logits + b * a.seq_stride + t * a.row_stride;
    const double lse = a.lse[row];
    const double H = a.g_entropy ? a.entropy[row] : 0.0;
    for (int64_t v = tid; v < a.vocab; v += kT64) {
        const double tt = x[v] * a.inv_t - lse;
        // (without an entropy gradient the factor is the constant -gsum: h * tt would be 0 * -inf at a -inf logit)
        out[v] = exp(tt) * (h != 0.0 ? -gsum - h * (tt + H) : -gsum) * a.inv_t;
    }
    __syncthreads();  // the one-hot terms are added by one lane after every softmax term of the row is stored
    if (tid == 0)
        for (int k = 0; k < a.n_index; ++k) {
            const int64_t idx = a.index[row * a.n_index + k];
            if (idx >= 0 && idx < a.vocab) out[idx] += a.g_logp[row * a.n_index + k] * a.inv_t;
        }
}

int check64(const char* what, const void* p, int64_t n_seq, int64_t rows_per_seq, int64_t vocab, int64_t seq_stride,
            int64_t row_stride) {
    TRLK_REQUIRE(n_seq >= 0 && rows_per_seq >= 0, TRLK_ERR_BAD_SHAPE, "%s: negative row count", what);
    TRLK_REQUIRE(vocab >= 1, TRLK_ERR_BAD_SHAPE, "%s: vocab must be >= 1 (got %lld)", what, (long long)vocab);
    TRLK_REQUIRE(n_seq * rows_per_seq < (int64_t(1) << 31), TRLK_ERR_BAD_SHAPE, "%s: too many rows", what);
    if (n_seq * rows_per_seq > 0) {
        TRLK_REQUIRE(p != nullptr, TRLK_ERR_NULL_POINTER, "%s: null data pointer", what);
        TRLK_REQUIRE(row_stride >= vocab || rows_per_seq <= 1, TRLK_ERR_BAD_STRIDE, "%s: row_stride %lld < vocab %lld (rows overlap)",
                     what, (long long)row_stride, (long long)vocab);
        TRLK_REQUIRE(seq_stride >= 0 && row_stride >= 0, TRLK_ERR_BAD_STRIDE, "%s: negative stride", what);
    }
    return TRLK_OK;
}

}  // namespace
}  // namespace trlk

using namespace trlk;

extern "C" int trlk_logp_entropy_fwd_f64(const double* d_logits, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                                         int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                                         double temperature, const uint8_t* d_row_mask, double* d_out_logp,
                                         double* d_out_entropy, double* d_out_lse, int32_t* d_error_flag,
                                         trlk_stream_t stream) {
    clear_error();
    if (int rc = check64("logp_entropy_fwd_f64: logits", d_logits, n_seq, rows_per_seq, vocab, seq_stride, row_stride)) return rc;
    TRLK_REQUIRE(n_index >= 0, TRLK_ERR_BAD_SHAPE, "logp_entropy_fwd_f64: n_index must be >= 0 (got %d)", n_index);
    TRLK_REQUIRE(temperature > 0.0 && temperature < INFINITY, TRLK_ERR_BAD_VALUE,
                 "logp_entropy_fwd_f64: temperature must be positive and finite (got %g)", temperature);
    const int64_t rows = n_seq * rows_per_seq;
    if (rows == 0) return TRLK_OK;
    TRLK_REQUIRE(n_index == 0 || (d_index != nullptr && d_out_logp != nullptr), TRLK_ERR_NULL_POINTER,
                 "logp_entropy_fwd_f64: index / out_logp pointer is null");
    TRLK_REQUIRE(n_index > 0 || d_out_entropy != nullptr || d_out_lse != nullptr, TRLK_ERR_NULL_POINTER,
                 "logp_entropy_fwd_f64: no output requested");
    Fwd64 a{d_logits, rows_per_seq, vocab, seq_stride, row_stride, d_index, n_index, 1.0 / temperature, d_row_mask,
            d_out_logp, d_out_entropy, d_out_lse, d_error_flag};
    hipLaunchKernelGGL(logp_entropy_fwd_f64_kernel, dim3((unsigned)rows), dim3(kT64), 0, static_cast<hipStream_t>(stream), a);
    return launch_status("logp_entropy_fwd_f64");
}

extern "C" int trlk_logp_entropy_bwd_f64(const double* d_logits, int64_t n_seq, int64_t rows_per_seq, int64_t vocab,
                                         int64_t seq_stride, int64_t row_stride, const int64_t* d_index, int32_t n_index,
                                         double temperature, const double* d_lse, const double* d_entropy,
                                         const double* d_g_logp, const double* d_g_entropy, double* d_dlogits,
                                         int64_t out_rows_per_seq, int64_t out_row_offset, int64_t out_seq_stride,
                                         int64_t out_row_stride, trlk_stream_t stream) {
    clear_error();
    if (int rc = check64("logp_entropy_bwd_f64: logits", d_logits, n_seq, rows_per_seq, vocab, seq_stride, row_stride)) return rc;
    if (int rc = check64("logp_entropy_bwd_f64: dlogits", d_dlogits, n_seq, out_rows_per_seq, vocab, out_seq_stride, out_row_stride))
        return rc;
    TRLK_REQUIRE(n_index >= 0, TRLK_ERR_BAD_SHAPE, "logp_entropy_bwd_f64: n_index must be >= 0 (got %d)", n_index);
    TRLK_REQUIRE(temperature > 0.0 && temperature < INFINITY, TRLK_ERR_BAD_VALUE,
                 "logp_entropy_bwd_f64: temperature must be positive and finite (got %g)", temperature);
    TRLK_REQUIRE(out_row_offset >= 0 && out_row_offset + rows_per_seq <= out_rows_per_seq, TRLK_ERR_BAD_SHAPE,
                 "logp_entropy_bwd_f64: input rows [%lld, %lld) do not fit the %lld output rows per sequence",
                 (long long)out_row_offset, (long long)(out_row_offset + rows_per_seq), (long long)out_rows_per_seq);
    const int64_t orows = n_seq * out_rows_per_seq;
    if (orows == 0) return TRLK_OK;
    if (n_seq * rows_per_seq > 0) {
        TRLK_REQUIRE(d_lse != nullptr, TRLK_ERR_NULL_POINTER, "logp_entropy_bwd_f64: lse pointer is null");
        TRLK_REQUIRE(n_index == 0 || (d_index != nullptr && d_g_logp != nullptr), TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd_f64: index / g_logp pointer is null");
        TRLK_REQUIRE((d_g_entropy == nullptr) == (d_entropy == nullptr), TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd_f64: g_entropy and entropy must be given together");
        TRLK_REQUIRE(n_index > 0 || d_g_entropy != nullptr, TRLK_ERR_NULL_POINTER,
                     "logp_entropy_bwd_f64: no upstream gradient given");
    }
    Bwd64 a{d_logits, rows_per_seq, vocab, seq_stride, row_stride, d_index, n_index, 1.0 / temperature, d_lse, d_entropy,
            d_g_logp, d_g_entropy, d_dlogits, out_rows_per_seq, out_row_offset, out_seq_stride, out_row_stride};
    hipLaunchKernelGGL(logp_entropy_bwd_f64_kernel, dim3((unsigned)orows), dim3(kT64), 0, static_cast<hipStream_t>(stream), a);
    return launch_status("logp_entropy_bwd_f64");
}
