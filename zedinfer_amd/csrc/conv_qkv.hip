// What stands between the q/k/v projection and attention in a mixer whose projections pass a short causal
// convolution over time: per token and in float32,
//
//   u = projection + bias                                             [q | k | v] channels, C in all
//   y_t[c] = sum_j taps[c][j] * u_(t - (taps-1) + j)[c]                 zeros before the sequence's start
//   q = y_q / rms(y_q) * w_q,  k = y_k / rms(y_k) * w_k                 one root mean square over ALL heads' channels
//   the first R dims of every head of q and k turn in pairs (i, i + R/2) by the step's angles
//   q -> q_out [n][heads * D];  k, v -> the paged cache at the token's slot (heads of D values; a head of fewer
//   dims is followed by zeros, so that one head size serves keys of `dim` and values of `vdim` dims)
//
// Rows of the entry's earlier tokens in this step come from the projection itself, rows before the step from the
// request's tail: the last taps - 1 rows of u (bias included), float32, [taps-1][C] in the request's state slot,
// zero for a fresh request (`zi_conv_tail` writes the new tail after this kernel has read the old one).
//
// One workgroup per token; the convolved channels pass through LDS.  Sums run in an order fixed by the sizes.
#include "zi_common.h"
#include "zi_api.h"

#define CQ_THREADS 256
#define CQ_MAX_CHANNELS 15360      // with the angles (at most a head of them) within 64 KB of LDS
#define CQ_MAX_TAPS 16

// One value of the projection: the sum of its `splits` partial sums (split s at proj + s * split_stride), in rising order.
template <typename TP>
__device__ __forceinline__ float cq_value(const TP* __restrict__ proj, int64_t ld, int splits, int64_t split_stride,
                                          int64_t row, int c) {
    const TP* p = proj + row * ld + c;
    float v = zi_load(p);
    int s = 1;
    for (; s + 4 <= splits; s += 4) {      // four loads in flight; the additions keep their order
        const float a = zi_load(p + s * split_stride), b = zi_load(p + (s + 1) * split_stride),
                    cc = zi_load(p + (s + 2) * split_stride), d = zi_load(p + (s + 3) * split_stride);
        v += a; v += b; v += cc; v += d;
    }
    for (; s < splits; ++s) v += zi_load(p + s * split_stride);
    return v;
}

// The convolved value of channel c of token t.  With the number of taps known at compile time (TAPS > 0) the taps'
// inputs (projection + bias, or the tail's rows) come back in `u`, the token's own last, so that the kernel can move
// the tail on without reading it again; with float32 rows that are no partial sums every input is one load whose
// address alone depends on where it comes from, so all are in flight together.  TAPS == 0: any number of taps, and
// `u[0]` is the token's own input.
template <typename TP, int TAPS>
__device__ __forceinline__ float cq_conv(const TP* __restrict__ proj, int64_t ld, int splits, int64_t split_stride,
                                         const float* __restrict__ bias, const float* __restrict__ conv_w,
                                         const float* __restrict__ tail, int t, int local, int c, int C, int taps,
                                         float* u) {
    const float bc = bias ? bias[c] : 0.f;
    if constexpr (TAPS > 0) {
        float wv[TAPS];
#pragma unroll
        for (int j = 0; j < TAPS; ++j) wv[j] = conv_w[(int64_t)c * TAPS + j];
        bool done = false;
        if constexpr (sizeof(TP) == 4) {
            if (splits == 1) {
#pragma unroll
                for (int j = 0; j < TAPS; ++j) {
                    const int li = local - (TAPS - 1) + j;
                    const float* src = li >= 0 ? (const float*)proj + (int64_t)(t - local + li) * ld + c
                                               : tail + (int64_t)(li + TAPS - 1) * C + c;
                    u[j] = *src;
                }
#pragma unroll
                for (int j = 0; j < TAPS; ++j)
                    if (local - (TAPS - 1) + j >= 0) u[j] += bc;
                done = true;
            }
        }
        if (!done) {
#pragma unroll
            for (int j = 0; j < TAPS; ++j) {
                const int li = local - (TAPS - 1) + j;
                u[j] = li >= 0 ? cq_value(proj, ld, splits, split_stride, t - local + li, c) + bc
                               : tail[(int64_t)(li + TAPS - 1) * C + c];
            }
        }
        float y = 0.f;
#pragma unroll
        for (int j = 0; j < TAPS; ++j) y += wv[j] * u[j];
        return y;
    } else {
        u[0] = cq_value(proj, ld, splits, split_stride, t, c) + bc;
        float y = conv_w[(int64_t)c * taps + taps - 1] * u[0];
        for (int j = 0; j + 1 < taps; ++j) {
            const int li = local - (taps - 1) + j;
            const float x = li >= 0 ? cq_value(proj, ld, splits, split_stride, t - local + li, c) + bc
                                    : tail[(int64_t)(li + taps - 1) * C + c];
            y += conv_w[(int64_t)c * taps + j] * x;
        }
        return y;
    }
}

template <typename TP, typename T, int TAPS, int THREADS>
__global__ void __launch_bounds__(THREADS)
conv_qkv_kernel(T* __restrict__ q_out, int64_t ldq, T* __restrict__ kcache, T* __restrict__ vcache,
                const TP* __restrict__ proj, int64_t ld, int splits, int64_t split_stride, const float* __restrict__ bias,
                const float* __restrict__ conv_w, float* __restrict__ state, int64_t state_stride, int move_tail,
                const float* __restrict__ q_norm,
                const float* __restrict__ k_norm, float eps, const float* __restrict__ table, int rot,
                const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ entry_start,
                const int32_t* __restrict__ entry_slot, const int32_t* __restrict__ slots, int64_t cache_slots, int nh,
                int nkv, int dim, int vdim, int D, int taps, int page_size) {
    extern __shared__ float y[];      // [C] the convolved channels, q and k already times their gains; then [rot] angles
    __shared__ float red[16];
    const int t = blockIdx.x, e = tok_seq[t], local = t - entry_start[e];
    const int Qd = nh * dim, Kd = nkv * dim, Vd = nkv * vdim, C = Qd + Kd + Vd;
    float* tail = state + (int64_t)entry_slot[e] * state_stride;
    const int slot = slots ? slots[t] : -1;
    float sq = 0.f, sk = 0.f;
    float* ang = y + C;      // (cos, sin) of the token's angles: the same for every head
    if (table)
        for (int i = threadIdx.x; i < rot; i += THREADS) ang[i] = table[(int64_t)t * rot + i];
    for (int c = threadIdx.x; c < C; c += THREADS) {
        float u[TAPS > 0 ? TAPS : 1];
        const float gain = c < Qd ? q_norm[c] : (c < Qd + Kd ? k_norm[c - Qd] : 1.f);
        const float v = cq_conv<TP, TAPS>(proj, ld, splits, split_stride, bias, conv_w, tail, t, local, c, C, taps, u);
        y[c] = v * gain;
        if (c < Qd) sq += v * v;
        else if (c < Qd + Kd) sk += v * v;
        // a step in which every entry brings one token: no other workgroup reads this entry's tail, and this thread
        // alone reads and writes channel c of it, so the tail moves on here (a token without a place in the cache is
        // padding and moves nothing)
        if (move_tail && slot >= 0 && taps > 1) {
            if constexpr (TAPS > 0) {
#pragma unroll
                for (int k = 0; k + 1 < TAPS; ++k) tail[(int64_t)k * C + c] = u[k + 1];
            } else {
                for (int k = 0; k + 2 < taps; ++k) tail[(int64_t)k * C + c] = tail[(int64_t)(k + 1) * C + c];
                tail[(int64_t)(taps - 2) * C + c] = u[0];
            }
        }
    }
    sq = zi_block_sum(sq, red);
    sk = zi_block_sum(sk, red);
    __syncthreads();
    const float rq = 1.f / sqrtf(sq / (float)Qd + eps), rk = 1.f / sqrtf(sk / (float)Kd + eps);
    const int half = rot / 2;
    // queries: every (head, dim of the padded head)
    for (int i = threadIdx.x; i < nh * D; i += THREADS) {
        const int h = i / D, x = i % D;
        float v = 0.f;
        if (x < dim) {
            const int c = h * dim + x;
            v = y[c] * rq;
            if (x < rot) {
                const int p = x < half ? x : x - half;
                const float cs = ang[2 * p], sn = ang[2 * p + 1];
                const float o = y[x < half ? c + half : c - half] * rq;
                v = x < half ? v * cs - o * sn : v * cs + o * sn;
            }
        }
        zi_store(q_out + (int64_t)t * ldq + i, v);
    }
    if (!kcache || slot < 0 || (int64_t)slot >= cache_slots) return;      // a token without a place in the cache stores nothing
    const int64_t page = slot / page_size, off = slot % page_size;
    for (int i = threadIdx.x; i < nkv * D; i += THREADS) {
        const int g = i / D, x = i % D;
        float v = 0.f;
        if (x < dim) {
            const int c = g * dim + x;
            v = y[Qd + c] * rk;
            if (x < rot) {
                const int p = x < half ? x : x - half;
                const float cs = ang[2 * p], sn = ang[2 * p + 1];
                const float o = y[Qd + (x < half ? c + half : c - half)] * rk;
                v = x < half ? v * cs - o * sn : v * cs + o * sn;
            }
        }
        zi_store(kcache + ((page * nkv + g) * page_size + off) * D + x, v);
    }
    for (int i = threadIdx.x; i < nkv * D; i += THREADS) {
        const int g = i / D, x = i % D;
        const float v = x < vdim ? y[Qd + Kd + g * vdim + x] : 0.f;
        zi_store(vcache + ((page * nkv + g) * D + x) * page_size + off, v);
    }
}

// `move_tail` (only for steps in which every entry brings one token): the kernel also writes the new tail, and
// zi_conv_tail is not needed.  `splits` > 1: proj comes as float32 partial sums [splits][n][ld].
extern "C" int zi_conv_qkv(void* q_out, int dt, int64_t ldq, void* kcache, void* vcache, const void* proj, int proj_dt,
                           int64_t ld, int splits, int64_t split_stride, const float* bias, const float* conv_w,
                           float* state, int64_t state_stride, int move_tail, const float* q_norm, const float* k_norm,
                           float eps, const float* table, int rot, int n,
                           const int32_t* tok_seq, const int32_t* entry_start, const int32_t* entry_slot,
                           const int32_t* slots, int64_t cache_slots, int nh, int nkv, int dim, int vdim, int D, int taps,
                           int page_size, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0 && dim > 0 && vdim > 0 && D >= dim && D >= vdim && taps >= 1 &&
                   taps <= CQ_MAX_TAPS && page_size > 0,
               "conv_qkv: bad sizes (heads %d/%d, dim %d, vdim %d, head size %d, taps %d)", nh, nkv, dim, vdim, D, taps);
    const int64_t C = (int64_t)nh * dim + (int64_t)nkv * dim + (int64_t)nkv * vdim;
    ZI_REQUIRE(C <= CQ_MAX_CHANNELS, "conv_qkv: %lld channels are more than %d", (long long)C, CQ_MAX_CHANNELS);
    ZI_REQUIRE((C + rot) * (int64_t)sizeof(float) <= 65000, "conv_qkv: channels and angles do not fit the workgroup's memory");
    ZI_REQUIRE(ld >= C && ldq >= (int64_t)nh * D, "conv_qkv: a row is too short");
    ZI_REQUIRE(state_stride >= (int64_t)(taps - 1) * C, "conv_qkv: the state row is too short");
    ZI_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim && (rot == 0 || table), "conv_qkv: %d rotated dims of %d", rot, dim);
    ZI_REQUIRE(eps > 0.f, "conv_qkv: eps must be positive");
    ZI_REQUIRE(!(kcache || vcache) || (slots && kcache && vcache && cache_slots > 0), "conv_qkv: a cache without slots");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || proj_dt == ZI_F32), "conv_qkv: partial sums are float32");
    ZI_REQUIRE(!move_tail || slots, "conv_qkv: moving the tail needs the tokens' slots");
    if (n == 0) return 0;
    const size_t lds = (size_t)(C + rot) * sizeof(float);
    // few tokens: workgroups of 1,024 threads, so that a thread walks few channels one after the other (with bfloat16
    // results only: the two sizes add the squares in different orders, and the float32 path keeps one order whatever
    // the step holds)
    const bool wide = n <= 512 && C > CQ_THREADS && dt == ZI_BF16;
#define ZI_CQ(TAPS, THREADS)                                                                                           \
    conv_qkv_kernel<TP, T, TAPS, THREADS><<<n, THREADS, lds, stream>>>(                                                \
        (T*)q_out, ldq, (T*)kcache, (T*)vcache, (const TP*)proj, ld, splits, split_stride, bias, conv_w, state,       \
        state_stride, move_tail, q_norm, k_norm, eps, table, rot, tok_seq, entry_start, entry_slot, slots, cache_slots, \
        nh, nkv, dim, vdim, D, taps, page_size)
#define ZI_CQ_TAPS(THREADS)                                                 \
    switch (taps) {                                                         \
        case 2: ZI_CQ(2, THREADS); break;                                   \
        case 3: ZI_CQ(3, THREADS); break;                                   \
        case 4: ZI_CQ(4, THREADS); break;                                   \
        default: ZI_CQ(0, THREADS); break;                                  \
    }
    ZI_DISPATCH_DTYPE(proj_dt, TP, ZI_DISPATCH_DTYPE(dt, T, {
        if (wide) { ZI_CQ_TAPS(1024) } else { ZI_CQ_TAPS(CQ_THREADS) }
    }));
#undef ZI_CQ_TAPS
#undef ZI_CQ
    return zi_check_launch("conv_qkv");
}

// The convolution's new tail: the last taps - 1 rows of u = projection + bias of the sequence so far, from this
// step's rows and, where the entry brought fewer, from the old tail.  A thread reads all it needs of the old tail
// before it writes.  With `slots` (every token's place in the cache, negative for tokens that have none), only an
// entry's own tokens count: those without a place stand behind them (padding that gives steps recurring shapes) and
// must not move the tail, and an entry that has none at all (it belongs to no request) leaves its slot's tail alone.
template <typename TP>
__global__ void __launch_bounds__(256)
conv_tail_kernel(float* __restrict__ state, int64_t state_stride, const TP* __restrict__ proj, int64_t ld, int splits,
                 int64_t split_stride, const float* __restrict__ bias, const int32_t* __restrict__ entry_start,
                 const int32_t* __restrict__ entry_len, const int32_t* __restrict__ entry_slot,
                 const int32_t* __restrict__ slots, int C, int taps) {
    const int e = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= C) return;
    const int start = entry_start[e];
    int len = entry_len[e];
    if (slots) {
        int lo = 0, hi = len;          // the first token without a place: the entry's own tokens come first
        while (lo < hi) {
            const int mid = (lo + hi) / 2;
            if (slots[start + mid] >= 0) lo = mid + 1;
            else hi = mid;
        }
        len = lo;
        if (len == 0) return;
    }
    float* tail = state + (int64_t)entry_slot[e] * state_stride;
    const float bc = bias ? bias[c] : 0.f;
    float keep[CQ_MAX_TAPS];
#pragma unroll
    for (int k = 0; k < CQ_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        const int li = len - (taps - 1) + k;
        keep[k] = li >= 0 ? cq_value(proj, ld, splits, split_stride, start + li, c) + bc : tail[(int64_t)(li + taps - 1) * C + c];
    }
#pragma unroll
    for (int k = 0; k < CQ_MAX_TAPS; ++k) {
        if (k >= taps - 1) break;
        tail[(int64_t)k * C + c] = keep[k];
    }
}

extern "C" int zi_conv_tail(float* state, int64_t state_stride, const void* proj, int proj_dt, int64_t ld, int splits,
                            int64_t split_stride, const float* bias, const int32_t* entry_start, const int32_t* entry_len,
                            const int32_t* entry_slot, const int32_t* slots, int entries, int channels, int taps,
                            hipStream_t stream) {
    ZI_REQUIRE(entries >= 0 && entries <= 65535 && channels > 0 && taps >= 1 && taps <= CQ_MAX_TAPS,
               "conv_tail: bad sizes (at most %d taps)", CQ_MAX_TAPS);
    ZI_REQUIRE(ld >= channels && state_stride >= (int64_t)(taps - 1) * channels, "conv_tail: a row is too short");
    ZI_REQUIRE(splits >= 1 && (splits == 1 || proj_dt == ZI_F32), "conv_tail: partial sums are float32");
    if (entries == 0 || taps == 1) return 0;
    ZI_DISPATCH_DTYPE(proj_dt, TP, {
        conv_tail_kernel<TP><<<dim3((channels + 255) / 256, entries), 256, 0, stream>>>(
            state, state_stride, (const TP*)proj, ld, splits, split_stride, bias, entry_start, entry_len, entry_slot, slots,
            channels, taps);
    });
    return zi_check_launch("conv_tail");
}
