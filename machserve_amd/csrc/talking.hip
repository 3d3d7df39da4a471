// Attention whose heads exchange scores before the softmax ("talking heads"), over the paged cache, for a
// window that keeps a request's first tokens, keys and values of different widths, a norm over the whole
// query and key projections, a rotation of the first part of a head, and values blended with another
// layer's.  One kernel finishes a row of the q/k/v product (norm, rotation, blend) and writes its key and
// value into their pages.  The attention itself runs on the matrix cores, 16 rows and every head a block for
// steps of many rows and one row a block for decoding, several blocks sharing a tile's keys where tiles are
// few (a last kernel merges their shares); and on the vector units, one row a block, for the head sizes and
// counts that kernel does not take.
//
// Scores, the exchange between heads, the softmax and every sum are 32-bit in every build; so are the norm's
// statistics, angles, cosines and sines.  The softmax weights are rounded to the element type only as an
// operand of the product with the values on the matrix cores (not in the 32-bit build, and not on the vector
// units).  A row's result depends on its own keys alone; which kernel runs, and how many blocks share a
// row's keys, follows from the step's shape, and the kernels differ in rounding only.
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

// ---- a tile of 16 rows on the matrix cores -------------------------------------------------
// A block takes rows [16 b, 16 b + 16) of the step, every head; wave w takes heads [w * HPW, (w + 1) * HPW).  Keys go by
// in tiles of NT * 16 positions.  Per tile: each wave computes S^T = K Q^T for its heads (lane l: keys (l / 16) * 4 + i
// of a 16-key tile, query l % 16), scales it and leaves it in LDS; after a barrier it reads, for each of its heads,
// every head's score of its own (key, query) pairs and mixes them by the exchange matrix in 32-bit; then the running
// softmax, in which a lane belongs to one query throughout, and O^T += V^T P^T, the weights rounded to the element
// type as an operand of that product (not at all in the 32-bit build).  Rows of several requests in one tile are
// taken request by request: the rows of the others are masked, which leaves their sums as they are.
constexpr float TK_NEG_BIG = -1.0e30f;

// e^x for the softmax of the tile kernel: the hardware's exponential in the two-byte builds (a few units in the last
// place of 32 bits, far below the rounding of the weights to the element type as operands), the library's in 32-bit
__device__ __forceinline__ float tk_exp(float x) {
#ifdef MS_ELEM_HALF
    return __expf(x);
#else
    return expf(x);
#endif
}

// 4 or 8 elements of one row that lie side by side, into elements at .. of a fragment
__device__ __forceinline__ void frag_set4(Frag& f, int at, const elem_t* p) {
#ifdef MS_ELEM_HALF
    const half4_t v = *reinterpret_cast<const half4_t*>(p);
#else
    const f32x4 v = *reinterpret_cast<const f32x4*>(p);
#endif
#pragma unroll
    for (int i = 0; i < 4; ++i) f.v[at + i] = v[i];
}

template <int HPW, int ND, int NT>
__global__ __launch_bounds__(512) void talking_attention_tile_kernel(TalkArgs a, const int* __restrict__ seq_q_len, int T, int n_split,
                                                                     float* __restrict__ part_o, float* __restrict__ part_ml, int tile_rows) {
    constexpr int NKS = 4, BK = NT * 16;  // heads of up to 128 numbers
    extern __shared__ float lds[];
    const int H = a.H, d = a.d, dv = a.dv, KV = a.KV, rep = H / KV, ps = a.ps;
    // [H][NT][64 lanes][4]: a lane reads what the same lane of the wave that owns head g wrote (both hold the same
    // (key, query) pairs), so a wave's 64 lanes always touch 1,024 consecutive bytes: no two of them meet in a bank
    float* raw = lds;
    float* talk_s = raw + (size_t)H * 16 * NT * 16;  // [H][H]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r16 = lane & 15, grp = lane >> 4;
    // tile_rows = 16: a tile of the step's rows; 1: one row a block, the tile's other fifteen queries idle (decoding: the
    // rows belong to different requests, which a tile would take one after the other)
    const int r0 = blockIdx.x * tile_rows, r_end = min(r0 + tile_rows, T);
    const int my_row = min(r0 + r16, r_end - 1);
    const int h0 = wave * HPW;
    const bool active = h0 < H;  // a wave beyond the heads only keeps the barriers
    if (a.talk)
        for (int i = tid; i < H * H; i += blockDim.x) talk_s[i] = a.talk[i];
    float m_run[HPW], l_run[HPW];
    f32x4 acc[HPW][ND];
    Frag qf[HPW][NKS];  // the rows' queries: asked for once
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
        m_run[hh] = TK_NEG_BIG;
        l_run[hh] = 0.f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) acc[hh][dt] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const int d0 = ks * 32 + grp * 8;
            qf[hh][ks] = (h0 + hh < H && d0 < d) ? frag_load(a.q + ((size_t)my_row * H + h0 + hh) * d + d0) : frag_zero();
        }
    }
    const int kv0 = min(h0, H - 1) / rep;  // the key/value head of the wave's first head
    int s = seq_of_row(r0, a.seq_q_start, a.S);
    for (; s < a.S && a.seq_q_start[s] < r_end; ++s) {
        const int q0 = a.seq_q_start[s], qn = seq_q_len[s], p0 = a.seq_pos0[s];
        const int ra = max(r0, q0), rb = min(r_end, q0 + qn);  // this request's rows in the tile
        if (ra >= rb) continue;
        const int p_lo = p0 + (ra - q0), p_hi = p0 + (rb - 1 - q0);
        const bool mine = r0 + r16 >= ra && r0 + r16 < rb;
        const int pos = p0 + (r0 + r16 - q0);
        const int lo = a.window > 0 ? max(0, p_lo - a.window + 1) : 0;
        const int n_first = min(a.keep_first, lo);
        const int* table = a.block_table + (size_t)s * a.table_stride;
        const int a_end = (n_first + BK - 1) / BK;  // tiles of the first tokens: [0, a_end)
        const int b_begin = max(a_end, lo / BK), b_end = p_hi / BK + 1;
        const int all_tiles = a_end + (b_end - b_begin);
        // block (b, y) takes the y-th share of the tiles; the shares are merged by talking_merge_kernel
        const int per = (all_tiles + n_split - 1) / n_split;
        const int it_begin = blockIdx.y * per, n_tiles = min(all_tiles, it_begin + per);
        if (it_begin >= n_tiles) continue;  // the same for every thread of the block
        auto tile_pos = [&](int it) { return (it < a_end ? it : b_begin + (it - a_end)) * BK; };
        auto pages_of = [&](int kt0, int* page) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int lp = (kt0 + nt * 16) / ps;
                page[nt] = lp < a.table_stride ? table[lp] : -1;
            }
        };
        auto load_k = [&](int kvh, const int* page, int kt0, Frag (&kf)[NT][NKS]) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const int pg = max(page[nt], 0), off = (kt0 + nt * 16) % ps;
                const elem_t* krow = a.kpool + (((size_t)pg * KV + kvh) * ps + off + r16) * d;
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) {
                    const int d0 = ks * 32 + grp * 8;
                    kf[nt][ks] = d0 < d ? frag_load(krow + d0) : frag_zero();
                }
            }
        };
        auto load_v = [&](int kvh, const int* page, int kt0, Frag (&vf)[ND]) {
#pragma unroll
            for (int dt = 0; dt < ND; ++dt) {
                const int e = dt * 16 + r16;
                vf[dt] = frag_zero();
                if (e < dv) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const int pg = max(page[nt], 0), off = (kt0 + nt * 16) % ps + grp * 4;
                        frag_set4(vf[dt], nt * 4, a.vpool + (((size_t)pg * KV + kvh) * dv + e) * ps + off);
                    }
                }
            }
        };
        int page[NT], page_n[NT];
        Frag kf[NT][NKS], kf_n[NT][NKS], vf[ND];
        if (active) {
            pages_of(tile_pos(it_begin), page);
            load_k(kv0, page, tile_pos(it_begin), kf);
        }
        for (int it = it_begin; it < n_tiles; ++it) {
            const int kt0 = tile_pos(it);
            if (active) {
                // this tile's values and the next tile's keys are asked for now and used later
                load_v(kv0, page, kt0, vf);
                if (it + 1 < n_tiles) {
                    pages_of(tile_pos(it + 1), page_n);
                    load_k(kv0, page_n, tile_pos(it + 1), kf_n);
                }
                // ---- raw scores of this wave's heads
                int kv_have = kv0;
#pragma unroll
                for (int hh = 0; hh < HPW; ++hh) {
                    const int h = h0 + hh;
                    if (h >= H) break;
                    if (h / rep != kv_have) {
                        kv_have = h / rep;
                        load_k(kv_have, page, kt0, kf);
                    }
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        f32x4 sc = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
                        for (int ks = 0; ks < NKS; ++ks)
                            if (ks * 32 < d) mma_16x16x32(sc, kf[nt][ks], qf[hh][ks]);
                        *reinterpret_cast<f32x4*>(raw + (((size_t)h * NT + nt) * 64 + lane) * 4) = sc * a.scale;
                    }
                }
            }
            __syncthreads();
            if (active) {
                // ---- exchange, softmax, values
                int v_have = kv0;
#pragma unroll
                for (int hh = 0; hh < HPW; ++hh) {
                    const int h = h0 + hh;
                    if (h >= H) break;
                    if (h / rep != v_have) {
                        v_have = h / rep;
                        load_v(v_have, page, kt0, vf);
                    }
                    f32x4 mixed[NT];
                    if (a.talk) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt) mixed[nt] = (f32x4){0.f, 0.f, 0.f, 0.f};
                        for (int g = 0; g < H; ++g) {
                            const float w = talk_s[h * H + g];
#pragma unroll
                            for (int nt = 0; nt < NT; ++nt)
                                mixed[nt] += w * *reinterpret_cast<const f32x4*>(raw + (((size_t)g * NT + nt) * 64 + lane) * 4);
                        }
                    } else {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
                            mixed[nt] = *reinterpret_cast<const f32x4*>(raw + (((size_t)h * NT + nt) * 64 + lane) * 4);
                    }
                    bool ok[NT][4];
                    float tmax = TK_NEG_BIG;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const int key = kt0 + nt * 16 + grp * 4 + i;
                            ok[nt][i] = mine && page[nt] >= 0 && key <= pos && (a.window <= 0 || pos - key < a.window || key < a.keep_first);
                            if (ok[nt][i]) tmax = fmaxf(tmax, mixed[nt][i]);
                        }
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
                    const float m_new = fmaxf(m_run[hh], tmax);
                    float psum = 0.f;
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float p = ok[nt][i] ? tk_exp(mixed[nt][i] - m_new) : 0.f;
                            mixed[nt][i] = p;
                            psum += p;
                        }
                    psum += __shfl_xor(psum, 16, WAVE);
                    psum += __shfl_xor(psum, 32, WAVE);
                    // where no row's maximum rose the factor is exactly one: after the first tiles that is the rule
                    const bool rose = __any(m_new > m_run[hh]);
                    const float alpha = rose ? tk_exp(m_run[hh] - m_new) : 1.0f;
                    l_run[hh] = l_run[hh] * alpha + psum;
                    m_run[hh] = m_new;
                    Frag pf;
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        pf.v[i] = from_f32<elem_t>(mixed[0][i]);
                        pf.v[4 + i] = from_f32<elem_t>(NT > 1 ? mixed[NT - 1][i] : 0.f);
                    }
                    if (rose) {
#pragma unroll
                        for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                            for (int i = 0; i < 4; ++i) acc[hh][dt][i] *= alpha;
                    }
#pragma unroll
                    for (int dt = 0; dt < ND; ++dt) mma_16x16x32(acc[hh][dt], vf[dt], pf);
                }
            }
            __syncthreads();
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                page[nt] = page_n[nt];
#pragma unroll
                for (int ks = 0; ks < NKS; ++ks) kf[nt][ks] = kf_n[nt][ks];
            }
        }
    }
    // O^T: lane holds value columns dt * 16 + grp * 4 + i of query r16
    if (r0 + r16 < r_end && active) {
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
            const int h = h0 + hh;
            if (h >= H) break;
            if (n_split > 1) {  // this share's maximum, sum and unnormalised output
                const size_t at = ((size_t)(r0 + r16) * n_split + blockIdx.y) * H + h;
                if (grp == 0) {
                    part_ml[2 * at] = m_run[hh];
                    part_ml[2 * at + 1] = l_run[hh];
                }
#pragma unroll
                for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int e = dt * 16 + grp * 4 + i;
                        if (e < dv) part_o[at * dv + e] = acc[hh][dt][i];
                    }
                continue;
            }
            const float inv = 1.0f / l_run[hh];
            elem_t* dst = a.out + ((size_t)(r0 + r16) * H + h) * dv;
#pragma unroll
            for (int dt = 0; dt < ND; ++dt)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int e = dt * 16 + grp * 4 + i;
                    if (e < dv) dst[e] = from_f32<elem_t>(acc[hh][dt][i] * inv);
                }
        }
    }
}

// ---- one row a block, its keys cut over several blocks ------------------------------------------
// For decoding: block (t, y) takes the y-th share of the 64-position tiles that row t sees, with 16-byte loads of keys
// and values, and leaves a running maximum, sum and unnormalised output per head; a second kernel merges the shares
// (one share: the block normalises and writes the output itself).  Needs head sizes that are multiples of 8 and pages
// of a multiple of 16 positions.
constexpr int TK_MAX_REP = 16;

__device__ __forceinline__ void load8(const elem_t* p, float* out) {
    const Frag f = frag_load(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) out[i] = to_f32(f.v[i]);
}

__global__ __launch_bounds__(256) void talking_attention_split_kernel(TalkArgs a, int n_split, float* __restrict__ part_o,
                                                                      float* __restrict__ part_ml) {
    extern __shared__ float lds[];
    const int H = a.H, d = a.d, dv = a.dv, KV = a.KV, rep = H / KV, ps = a.ps;
    float* qs = lds;                      // [H * d], scaled
    float* raw = qs + H * d;              // [H][64]
    float* mix = raw + H * TK_KEYS;       // [H][64]: mixed scores, then weights
    float* head_m = mix + H * TK_KEYS;
    float* head_l = head_m + H;
    float* head_a = head_l + H;
    int* page_of = reinterpret_cast<int*>(head_a + H);  // [4] pages of the tile's 16-position parts, -1: none
    float* talk_s = reinterpret_cast<float*>(page_of + 4);  // [H][H]
    const int t = blockIdx.x, y = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (a.talk)
        for (int i = tid; i < H * H; i += 256) talk_s[i] = a.talk[i];
    const int s = seq_of_row(t, a.seq_q_start, a.S);
    const int pos = a.seq_pos0[s] + (t - a.seq_q_start[s]);
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int n_first = min(a.keep_first, lo);
    const int a_end = (n_first + TK_KEYS - 1) / TK_KEYS;
    const int b_begin = max(a_end, lo / TK_KEYS), b_end = pos / TK_KEYS + 1;
    const int n_tiles = a_end + (b_end - b_begin);
    const int per = (n_tiles + n_split - 1) / n_split;
    const int it0 = y * per, it1 = min(n_tiles, it0 + per);
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
    for (int it = it0; it < it1; ++it) {
        const int kt0 = (it < a_end ? it : b_begin + (it - a_end)) * TK_KEYS;
        __syncthreads();
        if (tid < 4) {
            const int lp = (kt0 + tid * 16) / ps;
            page_of[tid] = lp < a.table_stride ? table[lp] : -1;
        }
        __syncthreads();
        // raw scores: an item is (key/value head, key); its heads share the key's row
        for (int item = tid; item < KV * TK_KEYS; item += 256) {
            const int kvh = item >> 6, jj = item & 63, key = kt0 + jj, page = page_of[jj >> 4];
            float sc[TK_MAX_REP];
#pragma unroll
            for (int r = 0; r < TK_MAX_REP; ++r) sc[r] = 0.f;
            if (page >= 0 && key <= pos) {
                const elem_t* kr = a.kpool + (((size_t)page * KV + kvh) * ps + key % ps) * d;
                for (int c0 = 0; c0 < d; c0 += 128) {  // 128 numbers of the key's row are asked for at once
                    Frag kf[16];
#pragma unroll
                    for (int c = 0; c < 16; ++c)
                        if (c0 + c * 8 < d) kf[c] = frag_load(kr + c0 + c * 8);
#pragma unroll
                    for (int c = 0; c < 16; ++c) {
                        if (c0 + c * 8 < d) {
                            float k8[8];
#pragma unroll
                            for (int e = 0; e < 8; ++e) k8[e] = to_f32(kf[c].v[e]);
#pragma unroll
                            for (int r = 0; r < TK_MAX_REP; ++r) {
                                if (r < rep) {
                                    const float* qr = qs + (kvh * rep + r) * d + c0 + c * 8;
#pragma unroll
                                    for (int e = 0; e < 8; ++e) sc[r] += qr[e] * k8[e];
                                }
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int r = 0; r < TK_MAX_REP; ++r)
                if (r < rep) raw[(kvh * rep + r) * TK_KEYS + jj] = sc[r];
        }
        __syncthreads();
        for (int item = tid; item < H * TK_KEYS; item += 256) {
            const int h = item >> 6, jj = item & 63, key = kt0 + jj;
            float sc;
            if (a.talk) {
                sc = 0.f;
                for (int g = 0; g < H; ++g) sc += talk_s[h * H + g] * raw[g * TK_KEYS + jj];
            } else {
                sc = raw[item];
            }
            const bool ok = page_of[jj >> 4] >= 0 && key <= pos && (a.window <= 0 || pos - key < a.window || key < a.keep_first);
            mix[item] = ok ? sc : -INFINITY;
        }
        __syncthreads();
        for (int h = wave; h < H; h += 4) {
            const float sc = mix[h * TK_KEYS + lane];
            const float m_old = head_m[h];
            const float m_new = fmaxf(m_old, wave_max(sc));
            const float p = (sc == -INFINITY || m_new == -INFINITY) ? 0.f : expf(sc - m_new);
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
#pragma unroll
        for (int i = 0; i < TK_MAX_OUT; ++i) {
            const int c = tid + i * 256;
            if (c < n_out) {
                const int h = c / dv, e = c - h * dv, kvh = h / rep;
                float sum = 0.f;
                Frag vf[8];  // the tile's 64 values of this column: asked for at once
#pragma unroll
                for (int sub = 0; sub < 4; ++sub) {
                    const int page = max(page_of[sub], 0);
                    const elem_t* vr = a.vpool + (((size_t)page * KV + kvh) * dv + e) * ps + (kt0 + sub * 16) % ps;
                    vf[2 * sub] = frag_load(vr);
                    vf[2 * sub + 1] = frag_load(vr + 8);
                }
                const float* w = mix + h * TK_KEYS;  // a weight of a part without a page is zero
#pragma unroll
                for (int f = 0; f < 8; ++f)
#pragma unroll
                    for (int k = 0; k < 8; ++k) sum += w[f * 8 + k] * to_f32(vf[f].v[k]);
                acc[i] = acc[i] * head_a[h] + sum;
            }
        }
    }
    __syncthreads();
    if (n_split == 1) {
#pragma unroll
        for (int i = 0; i < TK_MAX_OUT; ++i) {
            const int c = tid + i * 256;
            if (c < n_out) a.out[(size_t)t * n_out + c] = from_f32<elem_t>(acc[i] / head_l[c / dv]);
        }
        return;
    }
    float* po = part_o + ((size_t)t * n_split + y) * n_out;
#pragma unroll
    for (int i = 0; i < TK_MAX_OUT; ++i) {
        const int c = tid + i * 256;
        if (c < n_out) po[c] = acc[i];
    }
    float* pml = part_ml + ((size_t)t * n_split + y) * H * 2;
    for (int h = tid; h < H; h += 256) {
        pml[2 * h] = head_m[h];
        pml[2 * h + 1] = head_l[h];
    }
}

// out[t, h, :] = sum_y part_o[t, y, h, :] e^(m_y - M) / sum_y l_y e^(m_y - M), M = max_y m_y, the shares in order.
// A block is one (row, head): the shares' factors are worked out once, then every thread sums its columns over the
// shares with nothing between the loads.
__global__ __launch_bounds__(128) void talking_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                            elem_t* __restrict__ out, int n_split, int H, int dv) {
    __shared__ float fac[256];
    __shared__ float inv_l;
    const int t = blockIdx.x, h = blockIdx.y, n_out = H * dv;
    const float* ml = part_ml + (size_t)t * n_split * H * 2 + 2 * h;
    if (threadIdx.x < 64) {
        float M = -INFINITY;
        for (int y = threadIdx.x; y < n_split; y += 64) M = fmaxf(M, ml[(size_t)y * H * 2]);
        M = wave_max(M);
        float L = 0.f;
        for (int y = threadIdx.x; y < n_split; y += 64) {
            const float m = ml[(size_t)y * H * 2];
            const float f = (m == -INFINITY || m <= TK_NEG_BIG) ? 0.f : expf(m - M);
            fac[y] = f;
            L += ml[(size_t)y * H * 2 + 1] * f;
        }
        L = wave_sum(L);
        if (threadIdx.x == 0) inv_l = 1.0f / L;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < dv; e += 128) {
        const float* po = part_o + (size_t)t * n_split * n_out + (size_t)h * dv + e;
        float o = 0.f;
#pragma unroll 8
        for (int y = 0; y < n_split; ++y) o += po[(size_t)y * n_out] * fac[y];
        out[(size_t)t * n_out + (size_t)h * dv + e] = from_f32<elem_t>(o * inv_l);
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

// Whether the tile kernel takes these sizes (else the kernel of one row a block runs): head sizes that are multiples
// of 8 up to 128, at most 32 heads of at most 128 values (a multiple of 4), pages of a multiple of 16 positions.
extern "C" int ms_talking_tile_takes(int H, int KV, int d, int dv, int ps) {
    if (H < 1 || KV < 1 || H % KV || d % 8 || d > 128 || dv > 128 || dv < 1 || dv % 4 || ps % 16 || H > 32) return 0;
    const int nt = H <= 20 ? 2 : 1;
    return ((size_t)H * 16 * nt * 16 + (size_t)H * H) * sizeof(float) <= (size_t)TK_MAX_LDS;
}

template <int HPW, int ND>
static void launch_tile(const TalkArgs& a, const int* seq_q_len, int T, int NW, int n_split, float* part_o, float* part_ml, int tile_rows,
                        hipStream_t stream) {
    const int nt = a.H <= 20 ? 2 : 1;
    const size_t lds = ((size_t)a.H * 16 * nt * 16 + (size_t)a.H * a.H) * sizeof(float);
    const dim3 grid(ceil_div(T, tile_rows), n_split), block(NW * 64);
    if (nt == 2)
        hipLaunchKernelGGL((talking_attention_tile_kernel<HPW, ND, 2>), grid, block, lds, stream, a, seq_q_len, T, n_split, part_o, part_ml,
                           tile_rows);
    else
        hipLaunchKernelGGL((talking_attention_tile_kernel<HPW, ND, 1>), grid, block, lds, stream, a, seq_q_len, T, n_split, part_o, part_ml,
                           tile_rows);
}

extern "C" int ms_talking_attention_tiles(const void* q, const void* kpool, const void* vpool, const float* talk, const int* block_table,
                                          int table_stride, const int* seq_q_start, const int* seq_q_len, const int* seq_pos0, int S,
                                          void* out, int T, int H, int KV, int d, int dv, int ps, int window, int keep_first, float scale,
                                          int n_split, float* part_o, float* part_ml, int tile_rows, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0, "attention: empty problem");
    MS_REQUIRE(tile_rows == 16 || tile_rows == 1, "attention in tiles: tiles of %d rows", tile_rows);
    MS_REQUIRE(n_split >= 1 && n_split <= 256 && (n_split == 1 || (part_o && part_ml)), "attention in tiles: %d shares", n_split);
    MS_REQUIRE(ms_talking_tile_takes(H, KV, d, dv, ps), "attention in tiles: %d heads over %d, keys of %d, values of %d, pages of %d are not taken",
               H, KV, d, dv, ps);
    MS_REQUIRE(window >= 0 && keep_first >= 0, "attention: window %d, %d first tokens kept", window, keep_first);
    MS_REQUIRE(q && kpool && vpool && block_table && seq_q_start && seq_q_len && seq_pos0 && out, "attention: a buffer is missing");
    MS_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kpool) | reinterpret_cast<uintptr_t>(vpool)) & 15) == 0,
               "attention in tiles: operands must be 16-byte aligned");
    TalkArgs a{(const elem_t*)q, (const elem_t*)kpool, (const elem_t*)vpool, talk, block_table, table_stride, seq_q_start, seq_pos0,
               S, (elem_t*)out, H, KV, d, dv, ps, window, keep_first, scale};
    const int hpw = H <= 8 ? 1 : H <= 16 ? 2 : 4, nw = ceil_div(H, hpw), nd = ceil_div(dv, 16);
#define MS_TILE(HP, NDD) launch_tile<HP, NDD>(a, seq_q_len, T, nw, n_split, part_o, part_ml, tile_rows, stream)
#define MS_TILE_ND(HP)                      \
    do {                                    \
        if (nd <= 1) MS_TILE(HP, 1);        \
        else if (nd <= 2) MS_TILE(HP, 2);   \
        else if (nd <= 4) MS_TILE(HP, 4);   \
        else MS_TILE(HP, 8);                \
    } while (0)
    if (hpw == 1) MS_TILE_ND(1);
    else if (hpw == 2) MS_TILE_ND(2);
    else MS_TILE_ND(4);
#undef MS_TILE_ND
#undef MS_TILE
    if (int rc = check_launch("attention in tiles")) return rc;
    if (n_split > 1) {
        hipLaunchKernelGGL(talking_merge_kernel, dim3(T, H), dim3(128), 0, stream, part_o, part_ml, (elem_t*)out, n_split, H, dv);
        return check_launch("attention merge");
    }
    return 0;
}

// Whether the kernel whose blocks share a row's keys takes these sizes (else: one block a row, element by element).
extern "C" int ms_talking_split_takes(int H, int KV, int d, int dv, int ps) {
    if (H < 1 || KV < 1 || H % KV || H / KV > TK_MAX_REP || d % 8 || ps % 16 || H * dv > 256 * TK_MAX_OUT) return 0;
    return ((size_t)H * d + 2 * (size_t)H * TK_KEYS + 3 * (size_t)H + 4 + (size_t)H * H) * sizeof(float) <= (size_t)TK_MAX_LDS;
}

// part_o float [T, n_split, H * dv] and part_ml float [T, n_split, H, 2] are the shares' workspace (unused with one share).
extern "C" int ms_talking_attention_split(const void* q, const void* kpool, const void* vpool, const float* talk, const int* block_table,
                                          int table_stride, const int* seq_q_start, const int* seq_pos0, int S, void* out, int T, int H,
                                          int KV, int d, int dv, int ps, int window, int keep_first, float scale, int n_split,
                                          float* part_o, float* part_ml, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0, "attention: empty problem");
    MS_REQUIRE(ms_talking_split_takes(H, KV, d, dv, ps), "attention in shares: %d heads over %d, keys of %d, values of %d, pages of %d are not taken",
               H, KV, d, dv, ps);
    MS_REQUIRE(window >= 0 && keep_first >= 0, "attention: window %d, %d first tokens kept", window, keep_first);
    MS_REQUIRE(n_split >= 1 && n_split <= 256 && (n_split == 1 || (part_o && part_ml)), "attention in shares: %d shares", n_split);
    MS_REQUIRE(q && kpool && vpool && block_table && seq_q_start && seq_pos0 && out, "attention: a buffer is missing");
    MS_REQUIRE(((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(kpool) | reinterpret_cast<uintptr_t>(vpool)) & 15) == 0,
               "attention in shares: operands must be 16-byte aligned");
    TalkArgs a{(const elem_t*)q, (const elem_t*)kpool, (const elem_t*)vpool, talk, block_table, table_stride, seq_q_start, seq_pos0,
               S, (elem_t*)out, H, KV, d, dv, ps, window, keep_first, scale};
    const size_t lds = ((size_t)H * d + 2 * (size_t)H * TK_KEYS + 3 * (size_t)H + 4 + (size_t)H * H) * sizeof(float);
    hipLaunchKernelGGL(talking_attention_split_kernel, dim3(T, n_split), dim3(256), lds, stream, a, n_split, part_o, part_ml);
    if (int rc = check_launch("attention in shares")) return rc;
    if (n_split > 1) {
        hipLaunchKernelGGL(talking_merge_kernel, dim3(T, H), dim3(128), 0, stream, part_o, part_ml, (elem_t*)out, n_split, H, dv);
        return check_launch("attention merge");
    }
    return 0;
}
