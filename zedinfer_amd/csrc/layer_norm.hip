// Layer norm with gain and bias, and the arrangement that puts it on a sublayer's output:
//
//   y = (x - mean(x)) / sqrt(mean((x - mean)^2) + eps) * w + b          (float32 arithmetic throughout)
//
// x may come as `splits` terms (term s at x + s * split_stride: partial sums of a product cut along k, or the
// results of several sublayers), which are added in rising order first.  With `resid` (float32, in place) the
// normed row is added to the residual stream, resid += y, and `out` (when given) receives the new residual row
// in the output type: the rounded copy that the next sublayer's matrix products read.  Without `resid`, `out`
// receives y.
//
// One workgroup per row; a thread keeps its values of the row in registers (up to LN_PER * LN_THREADS columns),
// wider rows are read again from memory.  From 64 rows on and rows of at most 64 * LN_PER columns a wavefront takes
// a row and no barrier is needed.  Sums run in an order fixed by the row's width alone.
#include "zi_common.h"
#include "zi_api.h"

#define LN_THREADS 256
#define LN_PER 16

template <typename TX>
__device__ __forceinline__ float ln_value(const TX* __restrict__ xr, int splits, int64_t split_stride, int j) {
    float v = zi_load(xr + j);
    for (int s = 1; s < splits; ++s) v += zi_load(xr + s * split_stride + j);
    return v;
}

template <typename TX, typename TW, typename TO, int THREADS>
__global__ void __launch_bounds__(LN_THREADS)
layer_norm_kernel(TO* __restrict__ out, int64_t ldo, float* __restrict__ resid, const TX* __restrict__ x, int splits,
                  int64_t split_stride, int64_t ldx, const TW* __restrict__ w, const TW* __restrict__ b, int n, int H,
                  float eps) {
    __shared__ float red[16];
    // THREADS == 64: a wavefront per row, four rows a workgroup
    const int64_t row = THREADS == ZI_WAVE ? (int64_t)blockIdx.x * (LN_THREADS / ZI_WAVE) + threadIdx.x / ZI_WAVE : blockIdx.x;
    const int tid = THREADS == ZI_WAVE ? threadIdx.x % ZI_WAVE : threadIdx.x;
    if (row >= n) return;
    const TX* xr = x + row * ldx;
    const bool held = H <= LN_PER * THREADS;
    float v[LN_PER];
    float sum = 0.f;
    if (held) {
#pragma unroll
        for (int i = 0; i < LN_PER; ++i) {
            const int j = tid + i * THREADS;
            v[i] = j < H ? ln_value(xr, splits, split_stride, j) : 0.f;
            sum += v[i];
        }
    } else {
        for (int j = tid; j < H; j += THREADS) sum += ln_value(xr, splits, split_stride, j);
    }
    sum = THREADS == ZI_WAVE ? zi_wave_sum(sum) : zi_block_sum(sum, red);
    const float mean = sum / (float)H;
    float ss = 0.f;
    if (held) {
#pragma unroll
        for (int i = 0; i < LN_PER; ++i) {
            const int j = tid + i * THREADS;
            const float d = j < H ? v[i] - mean : 0.f;
            ss += d * d;
        }
    } else {
        for (int j = tid; j < H; j += THREADS) {
            const float d = ln_value(xr, splits, split_stride, j) - mean;
            ss += d * d;
        }
    }
    ss = THREADS == ZI_WAVE ? zi_wave_sum(ss) : zi_block_sum(ss, red);
    const float r = 1.f / sqrtf(ss / (float)H + eps);
    float* rr = resid ? resid + row * H : nullptr;
    TO* orow = out ? out + row * ldo : nullptr;
    if (held) {
#pragma unroll
        for (int i = 0; i < LN_PER; ++i) {
            const int j = tid + i * THREADS;
            if (j < H) {
                float y = (v[i] - mean) * r * zi_load(w + j) + zi_load(b + j);
                if (rr) {
                    y += rr[j];
                    rr[j] = y;
                }
                if (orow) zi_store(orow + j, y);
            }
        }
    } else {
        for (int j = tid; j < H; j += THREADS) {
            float y = (ln_value(xr, splits, split_stride, j) - mean) * r * zi_load(w + j) + zi_load(b + j);
            if (rr) {
                y += rr[j];
                rr[j] = y;
            }
            if (orow) zi_store(orow + j, y);
        }
    }
}

extern "C" int zi_layer_norm(void* out, int out_dt, int64_t ldo, float* resid, const void* x, int x_dt, int splits,
                             int64_t split_stride, int64_t ldx, const void* w, const void* b, int w_dt, int n, int hidden,
                             float eps, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && hidden > 0 && ldx >= hidden && splits >= 1, "layer_norm: bad sizes n=%d hidden=%d splits=%d", n,
               hidden, splits);
    ZI_REQUIRE(out || resid, "layer_norm: neither an output nor a residual stream");
    ZI_REQUIRE(!out || ldo >= hidden, "layer_norm: output rows are too short");
    ZI_REQUIRE(eps > 0.f, "layer_norm: eps must be positive");
    ZI_REQUIRE(w && b, "layer_norm: gain and bias are both needed");
    if (n == 0) return 0;
    const bool wave_rows = n >= 64 && hidden <= LN_PER * ZI_WAVE;
    ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
        if (wave_rows)
            layer_norm_kernel<TX, TW, TO, ZI_WAVE><<<(n + 3) / 4, LN_THREADS, 0, stream>>>(
                (TO*)out, ldo, resid, (const TX*)x, splits, split_stride, ldx, (const TW*)w, (const TW*)b, n, hidden, eps);
        else
            layer_norm_kernel<TX, TW, TO, LN_THREADS><<<n, LN_THREADS, 0, stream>>>(
                (TO*)out, ldo, resid, (const TX*)x, splits, split_stride, ldx, (const TW*)w, (const TW*)b, n, hidden, eps);
    })));
    return zi_check_launch("layer_norm");
}
