// The gated delta rule: a recurrent mixer whose state per head is a matrix S [dim][vdim], float32.
//
//   for every token, per head:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
//
// with q, k unit vectors (q also times dim^-1/2), beta in (0, 1) and the decay g in (0, 1).  q, k and v come out
// of a short causal convolution over time (per channel, `taps` taps, the last one the current token's) and SiLU.
// A request's state is S and, for the convolution, the last taps - 1 rows that entered it; both live in one
// float32 row per request slot: [heads][dim][vdim] first, then [taps - 1][channels].
//
// Everything here is float32 arithmetic.  Three launches a step: `zi_delta_prepare` (convolution, SiLU, unit
// vectors, beta, g, for every token at once), `zi_delta_conv_state` (the new tail of the convolution's input),
// `zi_delta_rule` (the recurrence, token by token within an entry, entries and heads and columns in parallel).
#include "zi_common.h"
#include "zi_api.h"

__device__ __forceinline__ float delta_silu(float z) { return z / (1.f + expf(-z)); }
__device__ __forceinline__ float delta_softplus(float z) { return z > 30.f ? z : log1pf(expf(z)); }

// proj [n][ld]: columns [q (kvh*dim) | k (kvh*dim) | v (heads*vdim) | gate (heads*vdim) | b (heads) | a (heads)].
// One workgroup per token.
template <typename TW>
__global__ void __launch_bounds__(256)
delta_prepare_kernel(float* __restrict__ qk, float* __restrict__ v, float* __restrict__ beta_g,
                     const float* __restrict__ proj, int64_t ld, const TW* __restrict__ conv_w,
                     const TW* __restrict__ a_log, const TW* __restrict__ dt_bias, const float* __restrict__ state,
                     int64_t state_stride, int64_t conv_off, const int32_t* __restrict__ tok_seq,
                     const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_slot, int heads,
                     int kvh, int dim, int vdim, int taps) {
    extern __shared__ float act[];      // [channels]
    const int t = blockIdx.x, e = tok_seq[t];
    const int local = t - entry_start[e];
    const int qkc = 2 * kvh * dim, C = qkc + heads * vdim;
    const float* tail = state + (int64_t)entry_slot[e] * state_stride + conv_off;      // [taps - 1][C]
    for (int c = threadIdx.x; c < C; c += blockDim.x) {
        float y = 0.f;
        for (int j = 0; j < taps; ++j) {
            const int li = local - (taps - 1) + j;
            const float x = li >= 0 ? proj[(int64_t)(t - local + li) * ld + c] : tail[(int64_t)(li + taps - 1) * C + c];
            y += zi_load(conv_w + (int64_t)c * taps + j) * x;
        }
        act[c] = delta_silu(y);
    }
    __syncthreads();
    const int lane = threadIdx.x % ZI_WAVE, wave = threadIdx.x / ZI_WAVE, waves = blockDim.x / ZI_WAVE;
    for (int hd = wave; hd < 2 * kvh; hd += waves) {       // the heads of q, then those of k
        float ss = 0.f;
        for (int d = lane; d < dim; d += ZI_WAVE) ss += act[hd * dim + d] * act[hd * dim + d];
        ss = zi_wave_sum(ss);
        const float r = (1.f / sqrtf(ss + 1e-6f)) * (hd < kvh ? 1.f / sqrtf((float)dim) : 1.f);
        for (int d = lane; d < dim; d += ZI_WAVE) qk[(int64_t)t * qkc + hd * dim + d] = act[hd * dim + d] * r;
    }
    for (int c = threadIdx.x; c < heads * vdim; c += blockDim.x) v[(int64_t)t * heads * vdim + c] = act[qkc + c];
    const float* row = proj + (int64_t)t * ld + C + heads * vdim;      // b, then a
    for (int h = threadIdx.x; h < heads; h += blockDim.x) {
        beta_g[(int64_t)t * 2 * heads + h] = 1.f / (1.f + expf(-row[h]));
        const float step = delta_softplus(row[heads + h] + zi_load(dt_bias + h));
        beta_g[(int64_t)t * 2 * heads + heads + h] = expf(-expf(zi_load(a_log + h)) * step);
    }
}

extern "C" int zi_delta_prepare(float* qk, float* v, float* beta_g, const float* proj, int64_t ld, int n,
                                const void* conv_w, const void* a_log, const void* dt_bias, int w_dt, const float* state,
                                int64_t state_stride, int64_t conv_off, const int32_t* tok_seq, const int32_t* entry_start,
                                const int32_t* entry_slot, int heads, int kvh, int dim, int vdim, int taps,
                                hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && kvh > 0 && heads % kvh == 0 && dim > 0 && vdim > 0 && taps >= 1,
               "delta_prepare: bad sizes");
    const int64_t C = 2LL * kvh * dim + (int64_t)heads * vdim;
    ZI_REQUIRE(ld >= C + (int64_t)heads * vdim + 2 * heads, "delta_prepare: row stride too small");
    ZI_REQUIRE(C * sizeof(float) <= 64 * 1024, "delta_prepare: %lld channels are more than a workgroup holds", (long long)C);
    ZI_REQUIRE(state_stride >= conv_off + (int64_t)(taps - 1) * C, "delta_prepare: the state row is too short");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(w_dt, TW, {
        delta_prepare_kernel<TW><<<n, 256, C * sizeof(float), stream>>>(
            qk, v, beta_g, proj, ld, (const TW*)conv_w, (const TW*)a_log, (const TW*)dt_bias, state, state_stride, conv_off,
            tok_seq, entry_start, entry_slot, heads, kvh, dim, vdim, taps);
    });
    return zi_check_launch("delta_prepare");
}

// The convolution's new tail: the last taps - 1 rows of the sequence so far, from this step's rows and, where the
// entry brought fewer, from the old tail.  A thread reads all it needs of the old tail before it writes.
#define DELTA_MAX_TAPS 16

__global__ void __launch_bounds__(256)
delta_conv_state_kernel(float* __restrict__ state, int64_t state_stride, int64_t conv_off,
                        const float* __restrict__ proj, int64_t ld, const int32_t* __restrict__ entry_start,
                        const int32_t* __restrict__ entry_len, const int32_t* __restrict__ entry_slot, int C, int taps) {
    const int e = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int start = entry_start[e], len = entry_len[e];
    float* tail = state + (int64_t)entry_slot[e] * state_stride + conv_off;
    float keep[DELTA_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < DELTA_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        const int li = len - (taps - 1) + k;
        float x = 0.f;
        if (li >= 0) x = proj[(int64_t)(start + li) * ld + c];
        else x = tail[(int64_t)(li + taps - 1) * C + c];
        keep[k] = x;
    }
#pragma unroll
    for (int k = 0; k < DELTA_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        tail[(int64_t)k * C + c] = keep[k];
    }
}

extern "C" int zi_delta_conv_state(float* state, int64_t state_stride, int64_t conv_off, const float* proj, int64_t ld,
                                   const int32_t* entry_start, const int32_t* entry_len, const int32_t* entry_slot,
                                   int entries, int channels, int taps, hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && channels > 0 && taps >= 1 && taps - 1 <= DELTA_MAX_TAPS,
               "delta_conv_state: bad sizes (at most %d taps)", DELTA_MAX_TAPS + 1);
    ZI_REQUIRE(ld >= channels && state_stride >= conv_off + (int64_t)(taps - 1) * channels,
               "delta_conv_state: a row is too short");
    if (entries == 0 || taps == 1) return 0;
    delta_conv_state_kernel<<<dim3((channels + 255) / 256, entries), 256, 0, stream>>>(
        state, state_stride, conv_off, proj, ld, entry_start, entry_len, entry_slot, channels, taps);
    return zi_check_launch("delta_conv_state");
}

// The recurrence.  One wavefront per (entry, head, 16 columns of S): lane (col, part) holds rows part, part + 4,
// part + 8, ... of column col, so a dot product over dim is a quarter of it in every lane and two lane exchanges.
// The order of the additions is fixed by dim alone.  k and q of TOKS tokens at a time are brought into LDS.
#define DELTA_COLS 16
#define DELTA_PARTS 4
#define DELTA_TOKS 16

template <int R>      // rows a lane holds: dim <= 4 R
__global__ void __launch_bounds__(ZI_WAVE)
delta_rule_kernel(float* __restrict__ out, const float* __restrict__ qk, const float* __restrict__ v,
                  const float* __restrict__ beta_g, float* __restrict__ state, int64_t state_stride,
                  const int32_t* __restrict__ entry_start, const int32_t* __restrict__ entry_len,
                  const int32_t* __restrict__ entry_slot, int heads, int kvh, int dim, int vdim) {
    __shared__ float ks[DELTA_TOKS][4 * R], qs[DELTA_TOKS][4 * R];
    __shared__ float bg[DELTA_TOKS][2];
    const int e = blockIdx.z, h = blockIdx.y, lane = threadIdx.x;
    const int col = blockIdx.x * DELTA_COLS + lane % DELTA_COLS, part = lane / DELTA_COLS;
    const bool live = col < vdim;
    const int kh = h / (heads / kvh), qkc = 2 * kvh * dim;
    const int start = entry_start[e], len = entry_len[e];
    float* S = state + (int64_t)entry_slot[e] * state_stride + (int64_t)h * dim * vdim;
    float s[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = part + DELTA_PARTS * i;
        s[i] = (live && d < dim) ? S[(int64_t)d * vdim + col] : 0.f;
    }
    for (int t0 = 0; t0 < len; t0 += DELTA_TOKS) {
        const int cnt = len - t0 < DELTA_TOKS ? len - t0 : DELTA_TOKS;
        __syncthreads();
        for (int i = lane; i < cnt * dim; i += ZI_WAVE) {
            const int tt = i / dim, d = i % dim;
            const float* row = qk + (int64_t)(start + t0 + tt) * qkc;
            qs[tt][d] = row[kh * dim + d];
            ks[tt][d] = row[(kvh + kh) * dim + d];
        }
        if (lane < 2 * cnt) bg[lane / 2][lane % 2] = beta_g[(int64_t)(start + t0 + lane / 2) * 2 * heads + (lane % 2) * heads + h];
        __syncthreads();
        for (int tt = 0; tt < cnt; ++tt) {
            const int t = start + t0 + tt;
            const float beta = bg[tt][0], g = bg[tt][1];
            const float vv = live ? v[((int64_t)t * heads + h) * vdim + col] : 0.f;
            float dot = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const int d = part + DELTA_PARTS * i;
                s[i] *= g;
                if (d < dim) dot += s[i] * ks[tt][d];
            }
            dot += __shfl_xor(dot, 16, ZI_WAVE);
            dot += __shfl_xor(dot, 32, ZI_WAVE);
            const float u = beta * (vv - dot);
            float o = 0.f;
#pragma unroll
            for (int i = 0; i < R; ++i) {
                const int d = part + DELTA_PARTS * i;
                if (d < dim) {
                    s[i] += ks[tt][d] * u;
                    o += s[i] * qs[tt][d];
                }
            }
            o += __shfl_xor(o, 16, ZI_WAVE);
            o += __shfl_xor(o, 32, ZI_WAVE);
            if (live && part == 0) out[((int64_t)t * heads + h) * vdim + col] = o;
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int d = part + DELTA_PARTS * i;
        if (live && d < dim) S[(int64_t)d * vdim + col] = s[i];
    }
}

extern "C" int zi_delta_rule(float* out, const float* qk, const float* v, const float* beta_g, float* state,
                             int64_t state_stride, const int32_t* entry_start, const int32_t* entry_len,
                             const int32_t* entry_slot, int entries, int heads, int kvh, int dim, int vdim,
                             hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && heads > 0 && heads <= 65535 && kvh > 0 && heads % kvh == 0 && dim > 0 &&
               vdim > 0, "delta_rule: bad sizes");
    ZI_REQUIRE(dim <= 256, "delta_rule: dim %d is more than the 256 rows a wavefront holds", dim);
    ZI_REQUIRE(state_stride >= (int64_t)heads * dim * vdim, "delta_rule: the state row is too short");
    if (entries == 0) return 0;
    const dim3 grid((vdim + DELTA_COLS - 1) / DELTA_COLS, heads, entries);
#define ZI_DELTA_RULE(R)                                                                                         \
    delta_rule_kernel<R><<<grid, ZI_WAVE, 0, stream>>>(out, qk, v, beta_g, state, state_stride, entry_start,      \
                                                       entry_len, entry_slot, heads, kvh, dim, vdim)
    if (dim <= 32) ZI_DELTA_RULE(8);
    else if (dim <= 64) ZI_DELTA_RULE(16);
    else if (dim <= 128) ZI_DELTA_RULE(32);
    else ZI_DELTA_RULE(64);
#undef ZI_DELTA_RULE
    return zi_check_launch("delta_rule");
}

// o [rows][vdim] (a row per token and head) divided by its root mean square, times a weight [vdim], times
// SiLU of a gate read from gate[token][head * vdim + e] with row stride ld_gate.  A wavefront per row.
template <typename TO, typename TW>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(TO* __restrict__ out, const float* __restrict__ o, const TW* __restrict__ w,
                     const float* __restrict__ gate, int64_t ld_gate, int rows, int heads, int vdim, float eps) {
    const int lane = threadIdx.x % ZI_WAVE;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x / ZI_WAVE) + threadIdx.x / ZI_WAVE;
    if (row >= rows) return;
    const float* orow = o + row * vdim;
    float ss = 0.f;
    for (int j = lane; j < vdim; j += ZI_WAVE) ss += orow[j] * orow[j];
    ss = zi_wave_sum(ss);
    const float rstd = 1.f / sqrtf(ss / (float)vdim + eps);
    const float* grow = gate + (row / heads) * ld_gate + (row % heads) * vdim;
    for (int j = lane; j < vdim; j += ZI_WAVE)
        zi_store(out + row * vdim + j, orow[j] * rstd * zi_load(w + j) * delta_silu(grow[j]));
}

extern "C" int zi_gated_rmsnorm(void* out, int out_dt, const float* o, const void* w, int w_dt, const float* gate,
                                int64_t ld_gate, int n, int heads, int vdim, float eps, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && vdim > 0 && eps > 0.f && ld_gate >= (int64_t)heads * vdim, "gated_rmsnorm: bad sizes");
    if (n == 0) return 0;
    const int rows = n * heads;
    ZI_DISPATCH_DTYPE(out_dt, TO, ZI_DISPATCH_DTYPE(w_dt, TW, {
        gated_rmsnorm_kernel<TO, TW><<<(rows + 3) / 4, 256, 0, stream>>>((TO*)out, o, (const TW*)w, gate, ld_gate, rows,
                                                                         heads, vdim, eps);
    }));
    return zi_check_launch("gated_rmsnorm");
}
