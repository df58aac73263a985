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
// wider rows are read again from memory.  Rows of at most 64 * LN_PER columns are taken by a wavefront each and no
// barrier is needed.  Sums run in an order fixed by the row's width alone.
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

// ---- rows of H % 4 == 0 values, 16-byte aligned: everything a thread needs is loaded at once, in pieces of four ----
__device__ __forceinline__ float4 ln_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ln_load4(const zi_bf16* p) {
    const uint2 r = *reinterpret_cast<const uint2*>(p);
    return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                       __uint_as_float(r.y & 0xffff0000u));
}
__device__ __forceinline__ void ln_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void ln_store4(zi_bf16* p, float4 v) {
    uint2 r;
    r.x = zi_pack_bf16x2(v.x, v.y);
    r.y = zi_pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = r;
}

// Few rows, up to 16 terms: a workgroup per row, a thread owns IT groups of four consecutive values and issues
// every term's load before the first is used (the few-rows products leave up to a dozen partial sums).
template <typename TX, typename TW, typename TO, int IT>
__global__ void layer_norm_vec_kernel(TO* __restrict__ out, int64_t ldo, float* __restrict__ resid, const TX* __restrict__ x,
                                      int splits, int64_t split_stride, int64_t ldx, const TW* __restrict__ w,
                                      const TW* __restrict__ b, int H, float eps) {
    __shared__ float red[16];
    const int64_t row = blockIdx.x;
    float4 v[IT];
    float sum = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int j = (it * blockDim.x + threadIdx.x) * 4;
        v[it] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (j >= H) continue;
        const TX* xr = x + row * ldx + j;
        float4 d[16];
#pragma unroll
        for (int sp = 0; sp < 16; ++sp)
            d[sp] = (sp < splits) ? ln_load4(xr + (int64_t)sp * split_stride) : make_float4(0.f, 0.f, 0.f, 0.f);
        float4 t = d[0];
#pragma unroll
        for (int sp = 1; sp < 16; ++sp) { t.x += d[sp].x; t.y += d[sp].y; t.z += d[sp].z; t.w += d[sp].w; }
        v[it] = t;
        sum += (t.x + t.y) + (t.z + t.w);
    }
    const float mean = zi_block_sum(sum, red) / (float)H;
    float ss = 0.f;
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int j = (it * blockDim.x + threadIdx.x) * 4;
        if (j >= H) continue;
        v[it].x -= mean; v[it].y -= mean; v[it].z -= mean; v[it].w -= mean;
        ss += (v[it].x * v[it].x + v[it].y * v[it].y) + (v[it].z * v[it].z + v[it].w * v[it].w);
    }
    const float r = 1.f / sqrtf(zi_block_sum(ss, red) / (float)H + eps);
#pragma unroll
    for (int it = 0; it < IT; ++it) {
        const int j = (it * blockDim.x + threadIdx.x) * 4;
        if (j >= H) continue;
        const float4 wv = ln_load4(w + j), bv = ln_load4(b + j);
        float4 y = make_float4(v[it].x * r * wv.x + bv.x, v[it].y * r * wv.y + bv.y, v[it].z * r * wv.z + bv.z,
                               v[it].w * r * wv.w + bv.w);
        if (resid) {
            const float4 o = ln_load4(resid + row * H + j);
            y.x += o.x; y.y += o.y; y.z += o.z; y.w += o.w;
            ln_store4(resid + row * H + j, y);
        }
        if (out) ln_store4(out + row * ldo + j, y);
    }
}

// One or two terms: a wavefront per row, four rows a workgroup, no barrier.  A lane owns NV groups of four
// consecutive values, 256 values apart (every load instruction of the wavefront reads 1 KB of the row).
template <typename TX, typename TW, typename TO, int NV>
__global__ void __launch_bounds__(4 * ZI_WAVE)
layer_norm_rows_kernel(TO* __restrict__ out, int64_t ldo, float* __restrict__ resid, const TX* __restrict__ x, int splits,
                       int64_t split_stride, int64_t ldx, const TW* __restrict__ w, const TW* __restrict__ b, int n, int H,
                       float eps) {
    const int lane = threadIdx.x & (ZI_WAVE - 1), wave = threadIdx.x / ZI_WAVE;
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    if (row >= n) return;
    const TX* xr = x + row * ldx;
    const int64_t second = splits > 1 ? split_stride : 0;      // one term: read twice, counted once
    const float twice = splits > 1 ? 1.f : 0.f;
    float4 v[NV], d[NV], o[NV];
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4, jc = j < H ? j : 0;     // past the row: its start again, unused
        v[c] = ln_load4(xr + jc);
        d[c] = ln_load4(xr + second + jc);
        o[c] = resid ? ln_load4(resid + row * H + jc) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4;
        v[c].x += twice * d[c].x; v[c].y += twice * d[c].y; v[c].z += twice * d[c].z; v[c].w += twice * d[c].w;
        if (j < H) sum += (v[c].x + v[c].y) + (v[c].z + v[c].w);
    }
    const float mean = zi_wave_sum(sum) / (float)H;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4;
        v[c].x -= mean; v[c].y -= mean; v[c].z -= mean; v[c].w -= mean;
        if (j < H) ss += (v[c].x * v[c].x + v[c].y * v[c].y) + (v[c].z * v[c].z + v[c].w * v[c].w);
    }
    const float r = 1.f / sqrtf(zi_wave_sum(ss) / (float)H + eps);
#pragma unroll
    for (int c = 0; c < NV; ++c) {
        const int j = (c * ZI_WAVE + lane) * 4;
        if (j >= H) continue;
        const float4 wv = ln_load4(w + j), bv = ln_load4(b + j);
        float4 y = make_float4(v[c].x * r * wv.x + bv.x, v[c].y * r * wv.y + bv.y, v[c].z * r * wv.z + bv.z,
                               v[c].w * r * wv.w + bv.w);
        if (resid) {
            y.x += o[c].x; y.y += o[c].y; y.z += o[c].z; y.w += o[c].w;
            ln_store4(resid + row * H + j, y);
        }
        if (out) ln_store4(out + row * ldo + j, y);
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
    const bool aligned = hidden % 4 == 0 && ldx % 4 == 0 && split_stride % 4 == 0 && ((uintptr_t)x % 16) == 0 &&
                         ((uintptr_t)w % 16) == 0 && ((uintptr_t)b % 16) == 0 && ((uintptr_t)resid % 16) == 0 &&
                         ((uintptr_t)out % 16) == 0 && ldo % 4 == 0 && (x_dt == ZI_F32 || (ldx % 8 == 0 && ((uintptr_t)x % 8) == 0)) &&
                         !(x_dt == ZI_BF16 && splits > 1);
    // Which kernel runs depends on the row's width and the number of terms, never on the number of rows: a row's sums
    // are then the same whatever else is in the step.
    if (aligned && splits <= 2 && hidden <= 8192) {
        const int nv = (hidden + 4 * ZI_WAVE - 1) / (4 * ZI_WAVE);
        const int wgs = (n + 3) / 4;
#define ZI_LN_ROWS(NV)                                                                                                \
    layer_norm_rows_kernel<TX, TW, TO, NV><<<wgs, 4 * ZI_WAVE, 0, stream>>>(                                          \
        (TO*)out, ldo, resid, (const TX*)x, splits, split_stride, ldx, (const TW*)w, (const TW*)b, n, hidden, eps)
        ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
            if (nv <= 2) ZI_LN_ROWS(2);
            else if (nv <= 4) ZI_LN_ROWS(4);
            else if (nv <= 6) ZI_LN_ROWS(6);
            else if (nv <= 8) ZI_LN_ROWS(8);
            else if (nv <= 12) ZI_LN_ROWS(12);
            else if (nv <= 16) ZI_LN_ROWS(16);
            else if (nv <= 24) ZI_LN_ROWS(24);
            else ZI_LN_ROWS(32);
        })));
#undef ZI_LN_ROWS
        return zi_check_launch("layer_norm");
    }
    if (aligned && splits <= 16 && hidden <= 8192) {
        const int vecs = hidden / 4;
        const int it = vecs > 1024 ? 2 : 1;
        const int threads = ((vecs + it - 1) / it + ZI_WAVE - 1) / ZI_WAVE * ZI_WAVE;
        ZI_DISPATCH_DTYPE(x_dt, TX, ZI_DISPATCH_DTYPE(w_dt, TW, ZI_DISPATCH_DTYPE(out_dt, TO, {
            if (it == 1)
                layer_norm_vec_kernel<TX, TW, TO, 1><<<n, threads, 0, stream>>>(
                    (TO*)out, ldo, resid, (const TX*)x, splits, split_stride, ldx, (const TW*)w, (const TW*)b, hidden, eps);
            else
                layer_norm_vec_kernel<TX, TW, TO, 2><<<n, threads, 0, stream>>>(
                    (TO*)out, ldo, resid, (const TX*)x, splits, split_stride, ldx, (const TW*)w, (const TW*)b, hidden, eps);
        })));
        return zi_check_launch("layer_norm");
    }
    const bool wave_rows = hidden <= LN_PER * ZI_WAVE;
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
