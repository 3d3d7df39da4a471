// Attention whose heads exchange scores before the softmax ("talking heads"), over the paged cache, for a
// window that keeps a request's first tokens, keys and values of different widths, a norm over the whole
// query and key projections, a rotation of the first part of a head, and values blended with another
// layer's.  Two kernels: one finishes a row of the q/k/v product (norm, rotation, blend) and writes its key
// and value into their pages; the other is the attention of one row over the keys it sees.
//
// Scores, the exchange between heads, the softmax and the weighted sum of values are 32-bit in every build;
// so are the norm's statistics, angles, cosines and sines.  A row's result depends on its own keys alone
// and is summed in one fixed order: it does not depend on what else the step holds.
#include "common.cuh"

namespace ms {

__device__ __forceinline__ int seq_of_row(int t, const int* __restrict__ seq_q_start, int S) {
    int lo = 0, hi = S - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (seq_q_start[mid] <= t) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

struct PrepareArgs {
    const float* qkv;       // [n_partials, T, stride] partial sums of: q [H, d], k [KV, d], v [KV, dv]
    int n_partials;
    size_t partial_stride;
    int stride;
    const float* q_norm;    // [H * d] or null: no norm over the projection
    const float* k_norm;    // [KV * d] or null
    float eps;
    const int* positions;   // [T]
    const float* inv_freq;  // [rot / 2] or null: no rotation
    int rot;                // numbers of a head that are rotated, pairs (i, i + rot / 2)
    float cs_factor;        // what cosines and sines are multiplied by
    const float* v_other;   // [T, KV * dv] or null: values to blend with
    const float* v_lambda;  // one number: v = (1 - lambda) v + lambda v_other
    float* v_raw_out;       // [T, KV * dv] or null: receives the row's own values, before any blend
    const int* slot_map;    // [T] page * ps + offset
    elem_t* q_out;          // [T, H * d]
    elem_t* kpool;          // [pages, KV, ps, d]
    elem_t* vpool;          // [pages, KV, dv, ps]
    int H, KV, d, dv, ps;
};

__global__ __launch_bounds__(256) void prepare_kernel(PrepareArgs a) {
    __shared__ float scratch[4];
    extern __shared__ float lds[];
    float* row = lds;                 // stride floats
    float* cs = lds + a.stride;       // rot / 2 cosines, then rot / 2 sines
    const int t = blockIdx.x, nq = a.H * a.d, nk = a.KV * a.d, nv = a.KV * a.dv, half = a.rot / 2;
    float ssq = 0.f, ssk = 0.f;
    for (int c = threadIdx.x; c < nq + nk + nv; c += 256) {
        float v = 0.f;
        for (int p = 0; p < a.n_partials; ++p) v += a.qkv[p * a.partial_stride + (size_t)t * a.stride + c];
        row[c] = v;
        if (c < nq) ssq += v * v;
        else if (c < nq + nk) ssk += v * v;
    }
    for (int j = threadIdx.x; j < half; j += 256) {
        float c = 1.f, s = 0.f;
        if (a.inv_freq) sincosf((float)a.positions[t] * a.inv_freq[j], &s, &c);
        cs[j] = c * a.cs_factor;
        cs[half + j] = s * a.cs_factor;
    }
    ssq = block_sum<256>(ssq, scratch);
    ssk = block_sum<256>(ssk, scratch);
    const float inv_q = a.q_norm ? 1.0f / sqrtf(ssq / (float)nq + a.eps) : 1.0f;
    const float inv_k = a.k_norm ? 1.0f / sqrtf(ssk / (float)nk + a.eps) : 1.0f;
    __syncthreads();
    const int slot = a.slot_map[t];
    const int page = slot >= 0 ? slot / a.ps : 0, off = slot >= 0 ? slot % a.ps : 0;
    // q heads, then k heads; element i of a head: the rotated part in pairs, the rest as it is
    for (int c = threadIdx.x; c < nq + nk; c += 256) {
        const bool is_q = c < nq;
        const int cc = is_q ? c : c - nq;
        const int h = cc / a.d, i = cc - h * a.d;
        const float inv = is_q ? inv_q : inv_k;
        const float* nw = is_q ? a.q_norm : a.k_norm;
        const float* base = row + (is_q ? 0 : nq) + h * a.d;
        auto normed = [&](int e) { return base[e] * inv * (nw ? nw[h * a.d + e] : 1.0f); };
        float v;
        if (i < half) v = normed(i) * cs[i] - normed(i + half) * cs[half + i];
        else if (i < a.rot) v = normed(i) * cs[i - half] + normed(i - half) * cs[i];
        else v = normed(i);
        if (is_q) a.q_out[(size_t)t * nq + c] = from_f32<elem_t>(v);
        else if (slot >= 0) a.kpool[(((size_t)page * a.KV + h) * a.ps + off) * a.d + i] = from_f32<elem_t>(v);
    }
    const float lam = a.v_other ? a.v_lambda[0] : 0.f;
    for (int c = threadIdx.x; c < nv; c += 256) {
        float v = row[nq + nk + c];
        if (a.v_raw_out) a.v_raw_out[(size_t)t * nv + c] = v;
        if (a.v_other) v = (1.0f - lam) * v + lam * a.v_other[(size_t)t * nv + c];
        const int h = c / a.dv, e = c - h * a.dv;
        if (slot >= 0) a.vpool[(((size_t)page * a.KV + h) * a.dv + e) * a.ps + off] = from_f32<elem_t>(v);
    }
}

struct TalkArgs {
    const elem_t* q;       // [T, H * d], rotated
    const elem_t* kpool;   // [pages, KV, ps, d]
    const elem_t* vpool;   // [pages, KV, dv, ps]
    const float* talk;     // [H, H] or null: score_h = sum_g talk[h, g] score_g
    const int* block_table;
    int table_stride;
    const int* seq_q_start;
    const int* seq_pos0;
    int S;
    elem_t* out;           // [T, H * dv]
    int H, KV, d, dv, ps, window, keep_first;
    float scale;
};

constexpr int TK_KEYS = 64;     // keys of a tile
constexpr int TK_MAX_OUT = 32;  // outputs (head x value column) per thread: H * dv <= 256 * 32

// One block per row.  The keys a row at position p sees are [0, min(keep_first, lo)) and [lo, p] with
// lo = max(0, p - window + 1) (window 0: lo = 0); they are walked as one list, 64 at a time: raw scores of every
// head, the exchange between heads, a running softmax per head, and the weighted sum of values.
__global__ __launch_bounds__(256) void talking_attention_kernel(TalkArgs a) {
    extern __shared__ float lds[];
    const int H = a.H, d = a.d, dv = a.dv, rep = H / a.KV;
    float* qs = lds;                      // [H * d], scaled
    float* raw = qs + H * d;              // [H][64]
    float* mix = raw + H * TK_KEYS;       // [H][64]: mixed scores, then weights
    float* head_m = mix + H * TK_KEYS;    // [H] running maximum
    float* head_l = head_m + H;           // [H] running sum
    float* head_a = head_l + H;           // [H] factor of this tile for what was summed before
    int* key_at = reinterpret_cast<int*>(head_a + H);  // [64] page * ps + offset of the tile's keys, -1: none
    const int t = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int s = seq_of_row(t, a.seq_q_start, a.S);
    const int pos = a.seq_pos0[s] + (t - a.seq_q_start[s]);
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int n_first = min(a.keep_first, lo);
    const int n_vis = n_first + (pos - lo + 1);
    const int* table = a.block_table + (size_t)s * a.table_stride;
    for (int c = tid; c < H * d; c += 256) qs[c] = to_f32(a.q[(size_t)t * H * d + c]) * a.scale;
    for (int h = tid; h < H; h += 256) {
        head_m[h] = -INFINITY;
        head_l[h] = 0.f;
    }
    float acc[TK_MAX_OUT];
#pragma unroll
    for (int i = 0; i < TK_MAX_OUT; ++i) acc[i] = 0.f;
    const int n_out = H * dv;
    for (int v0 = 0; v0 < n_vis; v0 += TK_KEYS) {
        __syncthreads();
        if (tid < TK_KEYS) {
            const int v = v0 + tid;
            int at = -1;
            if (v < n_vis) {
                const int j = v < n_first ? v : lo + (v - n_first);
                const int page = table[j / a.ps];
                at = page >= 0 ? page * a.ps + j % a.ps : -1;
            }
            key_at[tid] = at;
        }
        __syncthreads();
        // raw scores: every (head, key) of the tile
        for (int it = tid; it < H * TK_KEYS; it += 256) {
            const int g = it >> 6, jj = it & 63, at = key_at[jj];
            float sc = 0.f;
            if (at >= 0) {
                const elem_t* kr = a.kpool + (((size_t)(at / a.ps) * a.KV + g / rep) * a.ps + at % a.ps) * d;
                const float* qr = qs + g * d;
                for (int e = 0; e < d; ++e) sc += qr[e] * to_f32(kr[e]);
            }
            raw[it] = sc;
        }
        __syncthreads();
        // the exchange between heads
        for (int it = tid; it < H * TK_KEYS; it += 256) {
            const int h = it >> 6, jj = it & 63;
            float sc;
            if (a.talk) {
                sc = 0.f;
                for (int g = 0; g < H; ++g) sc += a.talk[h * H + g] * raw[g * TK_KEYS + jj];
            } else {
                sc = raw[it];
            }
            mix[it] = key_at[jj] >= 0 ? sc : -INFINITY;
        }
        __syncthreads();
        // running softmax: a wave takes heads wave, wave + 4, ...; a lane one key
        for (int h = wave; h < H; h += 4) {
            const float sc = mix[h * TK_KEYS + lane];
            const float m_old = head_m[h];
            const float m_new = fmaxf(m_old, wave_max(sc));
            const float p = sc == -INFINITY ? 0.f : expf(sc - m_new);
            const float sum = wave_sum(p);
            mix[h * TK_KEYS + lane] = p;
            if (lane == 0) {
                const float al = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
                head_a[h] = al;
                head_l[h] = head_l[h] * al + sum;
                head_m[h] = m_new;
            }
        }
        __syncthreads();
        // weighted sum of values: thread takes outputs tid, tid + 256, ...
#pragma unroll
        for (int i = 0; i < TK_MAX_OUT; ++i) {
            const int c = tid + i * 256;
            if (c < n_out) {
                const int h = c / dv, e = c - h * dv, kvh = h / rep;
                float sum = 0.f;
                const float* w = mix + h * TK_KEYS;
                for (int jj = 0; jj < TK_KEYS; ++jj) {
                    const int at = key_at[jj];
                    if (at >= 0) sum += w[jj] * to_f32(a.vpool[(((size_t)(at / a.ps) * a.KV + kvh) * dv + e) * a.ps + at % a.ps]);
                }
                acc[i] = acc[i] * head_a[h] + sum;
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < TK_MAX_OUT; ++i) {
        const int c = tid + i * 256;
        if (c < n_out) a.out[(size_t)t * n_out + c] = from_f32<elem_t>(acc[i] / head_l[c / dv]);
    }
}

}  // namespace ms

using namespace ms;

constexpr int TK_MAX_LDS = 64 * 1024;

// The most floats of a row of q, k and v that the first kernel holds in a block's LDS.
extern "C" int ms_talking_max_row() { return 15000; }

extern "C" int ms_talking_prepare(const float* qkv, int n_partials, int stride, const float* q_norm, const float* k_norm, float eps,
                                  const int* positions, const float* inv_freq, int rot, float cs_factor, const float* v_other,
                                  const float* v_lambda, float* v_raw_out, const int* slot_map, void* q_out, void* kpool,
                                  void* vpool, int T, int H, int KV, int d, int dv, int ps, hipStream_t stream) {
    MS_REQUIRE(T > 0 && H > 0 && KV > 0 && d > 0 && dv > 0 && ps > 0 && n_partials > 0, "attention rows: empty problem");
    MS_REQUIRE(stride >= (H + KV) * d + KV * dv && stride <= 15000, "attention rows: rows of %d for %d + %d heads of %d and %d values of %d",
               stride, H, KV, d, KV, dv);
    MS_REQUIRE(rot >= 0 && rot <= d && rot % 2 == 0, "attention rows: %d of %d numbers of a head are rotated", rot, d);
    MS_REQUIRE(qkv && positions && slot_map && q_out && kpool && vpool, "attention rows: a buffer is missing");
    MS_REQUIRE(!v_other || v_lambda, "attention rows: values to blend with, but no weight");
    PrepareArgs a{qkv, n_partials, (size_t)T * stride, stride, q_norm, k_norm, eps, positions, inv_freq, inv_freq ? rot : 0, cs_factor,
                  v_other, v_lambda, v_raw_out, slot_map, (elem_t*)q_out, (elem_t*)kpool, (elem_t*)vpool, H, KV, d, dv, ps};
    const size_t lds = (size_t)(stride + a.rot + 2) * sizeof(float);
    hipLaunchKernelGGL(prepare_kernel, dim3(T), dim3(256), lds, stream, a);
    return check_launch("attention rows");
}

extern "C" int ms_talking_attention(const void* q, const void* kpool, const void* vpool, const float* talk, const int* block_table,
                                    int table_stride, const int* seq_q_start, const int* seq_pos0, int S, void* out, int T, int H,
                                    int KV, int d, int dv, int ps, int window, int keep_first, float scale, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && H > 0 && KV > 0 && d > 0 && dv > 0 && ps > 0, "attention: empty problem");
    MS_REQUIRE(H % KV == 0, "attention: %d heads over %d key/value heads", H, KV);
    MS_REQUIRE(H * dv <= 256 * TK_MAX_OUT, "attention: %d heads of %d values exceed %d outputs a row", H, dv, 256 * TK_MAX_OUT);
    MS_REQUIRE(window >= 0 && keep_first >= 0, "attention: window %d, %d first tokens kept", window, keep_first);
    MS_REQUIRE(q && kpool && vpool && block_table && seq_q_start && seq_pos0 && out, "attention: a buffer is missing");
    const size_t lds = ((size_t)H * d + 2 * (size_t)H * TK_KEYS + 3 * (size_t)H + TK_KEYS) * sizeof(float);
    MS_REQUIRE(lds <= TK_MAX_LDS, "attention: %d heads of %d need %zu bytes of LDS, at most %d", H, d, lds, TK_MAX_LDS);
    TalkArgs a{(const elem_t*)q, (const elem_t*)kpool, (const elem_t*)vpool, talk, block_table, table_stride, seq_q_start, seq_pos0,
               S, (elem_t*)out, H, KV, d, dv, ps, window, keep_first, scale};
    hipLaunchKernelGGL(talking_attention_kernel, dim3(T), dim3(256), lds, stream, a);
    return check_launch("attention");
}
