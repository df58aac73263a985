// Latent attention: every token keeps one short latent c [rank] (RMS-normed) and one rotated key part kr [rot]
// that all heads share; a head's key is (W_uk c, kr) and its value W_uv c.  Nothing but c and kr is kept, and
// nothing else is ever made: the query's unrotated part is carried through W_uk once (qa = W_uk^T q), so that
//   score_j = (qa . c_j + q_rot . kr_j) * scale,   o = W_uv sum_j P_j c_j,
// which is the same sum in another order.  Scores, softmax and both sums are float32.
//
// Cache layout of one layer: c [page][slot][rank], kr [page][slot][rot]; a token's slot s lies in page
// s / page_size at s % page_size, so both are flat arrays indexed by the slot.
//
// The rotation turns neighbouring pairs (2i, 2i + 1) by the step's table of (cos, sin) [n][rot / 2][2].
#include "zi_common.h"
#include "zi_api.h"

// ---- the rotation alone: the first `rot` dims of every head of x [n][heads * d], in place --------------------
template <typename T>
__global__ void rope_pairs_kernel(T* __restrict__ x, int64_t ld, const float* __restrict__ table, int n, int heads, int d,
                                  int rot) {
    const int half = rot / 2;
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (int64_t)n * heads * half) return;
    const int p = (int)(i % half), h = (int)((i / half) % heads);
    const int64_t t = i / ((int64_t)half * heads);
    T* at = x + t * ld + (int64_t)h * d + 2 * p;
    const float u = zi_load(at), v = zi_load(at + 1);
    const float c = table[(t * half + p) * 2], s = table[(t * half + p) * 2 + 1];
    zi_store(at, u * c - v * s);
    zi_store(at + 1, v * c + u * s);
}

extern "C" int zi_rope_pairs(void* x, int dt, int64_t ld, const float* table, int n, int heads, int d, int rot,
                             hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && d > 0 && rot >= 0 && rot % 2 == 0 && rot <= d && ld >= (int64_t)heads * d,
               "rope_pairs: bad sizes");
    const int64_t total = (int64_t)n * heads * (rot / 2);
    if (total == 0) return 0;
    ZI_REQUIRE(table, "rope_pairs: no table of angles");
    ZI_DISPATCH_DTYPE(dt, T, {
        rope_pairs_kernel<T><<<(unsigned)((total + 255) / 256), 256, 0, stream>>>((T*)x, ld, table, n, heads, d, rot);
    });
    return zi_check_launch("rope_pairs");
}

// ---- the new token's latent and rotated key part, normed, turned and stored ---------------------------------
template <typename T, typename TW>
__global__ void __launch_bounds__(256)
latent_store_kernel(const float* __restrict__ dkv, int64_t ld, const TW* __restrict__ norm_w, float eps,
                    const float* __restrict__ table, const int32_t* __restrict__ slots, T* __restrict__ c_cache,
                    T* __restrict__ kr_cache, int64_t cache_slots, int rank, int rot) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int slot = slots[t];
    if (slot < 0 || slot >= cache_slots) return;      // a token without a place (padding): the whole workgroup leaves
    const float* row = dkv + (int64_t)t * ld;
    float ss = 0.f;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) {
        const float v = zi_load(row + j);
        ss += v * v;
    }
    ss = zi_block_sum(ss, red);
    const float rstd = 1.0f / sqrtf(ss / (float)rank + eps);
    T* cr = c_cache + (int64_t)slot * rank;
    for (int j = threadIdx.x; j < rank; j += blockDim.x) zi_store(cr + j, zi_load(row + j) * rstd * zi_load(norm_w + j));
    T* kr = kr_cache + (int64_t)slot * rot;
    const float* tab = table + (int64_t)t * rot;      // [rot / 2][2]
    for (int i = threadIdx.x; i < rot / 2; i += blockDim.x) {
        const float u = zi_load(row + rank + 2 * i), v = zi_load(row + rank + 2 * i + 1);
        const float c = tab[2 * i], s = tab[2 * i + 1];
        zi_store(kr + 2 * i, u * c - v * s);
        zi_store(kr + 2 * i + 1, v * c + u * s);
    }
}

extern "C" int zi_latent_store(const float* dkv, int dt, int64_t ld, int n, const void* norm_w, int w_dt, float eps,
                               const float* table, const int32_t* slots, void* c_cache, void* kr_cache,
                               int64_t cache_slots, int rank, int rot, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && rank > 0 && rot >= 0 && rot % 2 == 0 && ld >= rank + rot, "latent_store: bad sizes");
    ZI_REQUIRE(eps > 0.f && cache_slots > 0, "latent_store: bad eps or cache");
    ZI_REQUIRE(rot == 0 || table, "latent_store: a rotated part needs the table of angles");
    if (n == 0) return 0;
    ZI_DISPATCH_DTYPE(dt, T, ZI_DISPATCH_DTYPE(w_dt, TW, {
        latent_store_kernel<T, TW><<<n, 256, 0, stream>>>(dkv, ld, (const TW*)norm_w, eps, table, slots,
                                                          (T*)c_cache, (T*)kr_cache, cache_slots, rank, rot);
    }));
    return zi_check_launch("latent_store");
}

// ---- queries: qa[t][h] = (W_uk[h]^T q_plain[t][h], turn(q_rot[t][h])), float32 ------------------------------
// One workgroup per (tile of QT tokens, head).  W_uk is [heads * dim][rank], row h * dim + d the d-th unrotated
// dimension of head h: for a fixed d the threads read neighbouring ranks.
#define LATENT_QT 8

template <typename T, typename TW>
__global__ void __launch_bounds__(256)
latent_query_kernel(float* __restrict__ qa, const T* __restrict__ q, int64_t ldq, const TW* __restrict__ w_uk,
                    const float* __restrict__ table, int n, int heads, int dim, int rank, int rot) {
    extern __shared__ float qs[];      // [LATENT_QT][dim]
    const int t0 = blockIdx.x * LATENT_QT, h = blockIdx.y;
    const int width = dim + rot, out_w = rank + rot;
    for (int i = threadIdx.x; i < LATENT_QT * dim; i += blockDim.x) {
        const int tt = i / dim, d = i % dim;
        qs[i] = t0 + tt < n ? zi_load(q + (int64_t)(t0 + tt) * ldq + (int64_t)h * width + d) : 0.f;
    }
    __syncthreads();
    const TW* w = w_uk + (int64_t)h * dim * rank;
    for (int r = threadIdx.x; r < rank; r += blockDim.x) {
        float acc[LATENT_QT];
#pragma unroll
        for (int tt = 0; tt < LATENT_QT; ++tt) acc[tt] = 0.f;
        for (int d = 0; d < dim; ++d) {
            const float wv = zi_load(w + (int64_t)d * rank + r);
#pragma unroll
            for (int tt = 0; tt < LATENT_QT; ++tt) acc[tt] += qs[tt * dim + d] * wv;
        }
#pragma unroll
        for (int tt = 0; tt < LATENT_QT; ++tt)
            if (t0 + tt < n) qa[((int64_t)(t0 + tt) * heads + h) * out_w + r] = acc[tt];
    }
    for (int i = threadIdx.x; i < LATENT_QT * (rot / 2); i += blockDim.x) {
        const int tt = i / (rot / 2), p = i % (rot / 2), t = t0 + tt;
        if (t >= n) continue;
        const T* qr = q + (int64_t)t * ldq + (int64_t)h * width + dim;
        const float u = zi_load(qr + 2 * p), v = zi_load(qr + 2 * p + 1);
        const float c = table[((int64_t)t * (rot / 2) + p) * 2], s = table[((int64_t)t * (rot / 2) + p) * 2 + 1];
        float* o = qa + ((int64_t)t * heads + h) * out_w + rank;
        o[2 * p] = u * c - v * s;
        o[2 * p + 1] = v * c + u * s;
    }
}

extern "C" int zi_latent_query(float* qa, const void* q, int dt, int64_t ldq, const void* w_uk, int w_dt,
                               const float* table, int n, int heads, int dim, int rank, int rot, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && heads <= 65535 && dim > 0 && rank > 0 && rot >= 0 && rot % 2 == 0,
               "latent_query: bad sizes");
    ZI_REQUIRE(ldq >= (int64_t)heads * (dim + rot), "latent_query: row stride too small");
    ZI_REQUIRE((size_t)LATENT_QT * dim * sizeof(float) <= 64 * 1024, "latent_query: dim %d is too large", dim);
    ZI_REQUIRE(rot == 0 || table, "latent_query: a rotated part needs the table of angles");
    if (n == 0) return 0;
    const dim3 grid((n + LATENT_QT - 1) / LATENT_QT, heads);
    ZI_DISPATCH_DTYPE(dt, T, ZI_DISPATCH_DTYPE(w_dt, TW, {
        latent_query_kernel<T, TW><<<grid, 256, LATENT_QT * dim * sizeof(float), stream>>>(
            qa, (const T*)q, ldq, (const TW*)w_uk, table, n, heads, dim, rank, rot);
    }));
    return zi_check_launch("latent_query");
}

// ---- attention over the cached latents: the plain kernel ----------------------------------------------------
// One wavefront per (token, head).  The token at position p sees the keys at [lo, p], lo = 0 or p - window + 1.
// Takes rank + rot up to 1024 and rank up to 1024, any page size, both storage types, prompts and decoded
// tokens alike; a token's result depends on its own position and keys only.
#define LATENT_MAX_Q 1088
#define LATENT_MAX_RANK 1024
#define LATENT_ACC (LATENT_MAX_RANK / ZI_WAVE)

template <typename T, int ACC>
__global__ void __launch_bounds__(ZI_WAVE)
latent_attention_kernel(float* __restrict__ out, const float* __restrict__ qa, const T* __restrict__ c_cache,
                        const T* __restrict__ kr_cache, const int32_t* __restrict__ tok_index,
                        const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tok_pos,
                        const int32_t* __restrict__ block_tables, int max_pages, int num_pages, int heads, int rank,
                        int rot, int page_size, int window, float scale) {
    __shared__ float qs[LATENT_MAX_Q];
    __shared__ float ps[ZI_WAVE];
    __shared__ int64_t place[ZI_WAVE];
    const int t = tok_index ? tok_index[blockIdx.x] : blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int p = tok_pos[t];
    const int32_t* bt = block_tables + (int64_t)tok_seq[t] * max_pages;
    const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
    const int qw = rank + rot;
    const float* qr = qa + ((int64_t)t * heads + h) * qw;
    for (int j = lane; j < qw; j += ZI_WAVE) qs[j] = qr[j];
    __syncthreads();

    float m = -INFINITY, l = 0.f;
    float acc[ACC];
#pragma unroll
    for (int i = 0; i < ACC; ++i) acc[i] = 0.f;
    for (int base = lo; base <= p; base += ZI_WAVE) {
        const int j = base + lane;
        bool valid = j <= p;
        float s = -INFINITY;
        int64_t at = -1;
        if (valid) {
            const int pi = j / page_size;
            const int page = pi < max_pages ? bt[pi] : -1;
            if (page < 0 || page >= num_pages) {
                valid = false;      // a hole in the table: never scheduled; stay in bounds
            } else {
                at = (int64_t)page * page_size + (j % page_size);
                const T* cr = c_cache + at * rank;
                const T* kr = kr_cache + at * rot;
                float dot = 0.f;
                for (int x = 0; x < rank; ++x) dot += qs[x] * zi_load(cr + x);
                for (int x = 0; x < rot; ++x) dot += qs[rank + x] * zi_load(kr + x);
                s = dot * scale;
            }
        }
        const float m_new = fmaxf(m, zi_wave_max(s));
        const float pj = valid ? expf(s - m_new) : 0.f;
        const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
        l = l * corr + zi_wave_sum(pj);
        ps[lane] = pj;
        place[lane] = at;
        __syncthreads();
        const int cnt = (p - base + 1 < ZI_WAVE) ? p - base + 1 : ZI_WAVE;
#pragma unroll
        for (int i = 0; i < ACC; ++i) acc[i] *= corr;
        for (int jj = 0; jj < cnt; ++jj) {
            const int64_t a = place[jj];
            if (a < 0) continue;
            const float pw = ps[jj];
            const T* cr = c_cache + a * rank;
#pragma unroll
            for (int i = 0; i < ACC; ++i) {
                const int x = lane + i * ZI_WAVE;
                if (x < rank) acc[i] += pw * zi_load(cr + x);
            }
        }
        m = m_new;
        __syncthreads();
    }
    float* orow = out + ((int64_t)t * heads + h) * rank;
    const float inv = 1.f / l;
#pragma unroll
    for (int i = 0; i < ACC; ++i) {
        const int x = lane + i * ZI_WAVE;
        if (x < rank) orow[x] = acc[i] * inv;
    }
}

extern "C" int zi_latent_attention(float* out, const float* qa, const void* c_cache, const void* kr_cache, int dt,
                                   int n_idx, const int32_t* tok_index, const int32_t* tok_seq, const int32_t* tok_pos,
                                   const int32_t* block_tables, int max_pages, int num_pages, int heads, int rank, int rot,
                                   int page_size, int window, float scale, hipStream_t stream) {
    ZI_REQUIRE(n_idx >= 0 && heads > 0 && heads <= 65535 && rank > 0 && rot >= 0 && page_size > 0 && max_pages > 0 &&
               num_pages > 0 && window >= 0, "latent_attention: bad sizes");
    ZI_REQUIRE(rank <= LATENT_MAX_RANK && rank + rot <= LATENT_MAX_Q,
               "latent_attention: rank %d + rot %d is more than this kernel holds", rank, rot);
    if (n_idx == 0) return 0;
    const dim3 grid(n_idx, heads);
#define ZI_LATENT_ATT(ACC)                                                                                            \
    latent_attention_kernel<T, ACC><<<grid, ZI_WAVE, 0, stream>>>(out, qa, (const T*)c_cache, (const T*)kr_cache,      \
        tok_index, tok_seq, tok_pos, block_tables, max_pages, num_pages, heads, rank, rot, page_size, window, scale)
    ZI_DISPATCH_DTYPE(dt, T, {
        if (rank <= 2 * ZI_WAVE) ZI_LATENT_ATT(2);
        else if (rank <= 4 * ZI_WAVE) ZI_LATENT_ATT(4);
        else if (rank <= 8 * ZI_WAVE) ZI_LATENT_ATT(8);
        else ZI_LATENT_ATT(LATENT_ACC);
    });
#undef ZI_LATENT_ATT
    return zi_check_launch("latent_attention");
}

// ---- values: out[t][h * vdim + e] = W_uv[h * vdim + e] . o[t][h] -----------------------------------------------
template <typename TO, typename TW>
__global__ void __launch_bounds__(256)
latent_value_kernel(TO* __restrict__ out, int64_t ldo, const float* __restrict__ o, const TW* __restrict__ w_uv, int n,
                    int heads, int vdim, int rank) {
    extern __shared__ float os[];      // [LATENT_QT][rank]
    const int t0 = blockIdx.x * LATENT_QT, h = blockIdx.y;
    for (int i = threadIdx.x; i < LATENT_QT * rank; i += blockDim.x) {
        const int tt = i / rank, r = i % rank;
        os[i] = t0 + tt < n ? o[((int64_t)(t0 + tt) * heads + h) * rank + r] : 0.f;
    }
    __syncthreads();
    // a wavefront per output dimension: its lanes share the row of W_uv
    const int lane = threadIdx.x % ZI_WAVE, wave = threadIdx.x / ZI_WAVE, waves = blockDim.x / ZI_WAVE;
    for (int e = wave; e < vdim; e += waves) {
        const TW* w = w_uv + ((int64_t)h * vdim + e) * rank;
        float acc[LATENT_QT];
#pragma unroll
        for (int tt = 0; tt < LATENT_QT; ++tt) acc[tt] = 0.f;
        for (int r = lane; r < rank; r += ZI_WAVE) {
            const float wv = zi_load(w + r);
#pragma unroll
            for (int tt = 0; tt < LATENT_QT; ++tt) acc[tt] += os[tt * rank + r] * wv;
        }
#pragma unroll
        for (int tt = 0; tt < LATENT_QT; ++tt) {
            const float v = zi_wave_sum(acc[tt]);
            if (lane == 0 && t0 + tt < n) zi_store(out + (int64_t)(t0 + tt) * ldo + (int64_t)h * vdim + e, v);
        }
    }
}

extern "C" int zi_latent_value(void* out, int out_dt, int64_t ldo, const float* o, const void* w_uv, int w_dt, int n,
                               int heads, int vdim, int rank, hipStream_t stream) {
    ZI_REQUIRE(n >= 0 && heads > 0 && heads <= 65535 && vdim > 0 && rank > 0, "latent_value: bad sizes");
    ZI_REQUIRE(ldo >= (int64_t)heads * vdim, "latent_value: row stride too small");
    ZI_REQUIRE((size_t)LATENT_QT * rank * sizeof(float) <= 64 * 1024, "latent_value: rank %d is too large", rank);
    if (n == 0) return 0;
    const dim3 grid((n + LATENT_QT - 1) / LATENT_QT, heads);
    ZI_DISPATCH_DTYPE(out_dt, TO, ZI_DISPATCH_DTYPE(w_dt, TW, {
        latent_value_kernel<TO, TW><<<grid, 256, LATENT_QT * rank * sizeof(float), stream>>>(
            (TO*)out, ldo, o, (const TW*)w_uv, n, heads, vdim, rank);
    }));
    return zi_check_launch("latent_value");
}
