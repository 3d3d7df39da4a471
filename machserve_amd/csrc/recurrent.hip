// Mixers whose memory is a state of fixed size per request: the short causal convolution and the selective
// scan of a Mamba layer, and linear attention with a decay per head ("lightning" attention), with the gated
// norm that follows it.
//
// A step's rows are the tokens of several requests, each request's rows contiguous and in order
// (seq_q_start, seq_q_len); a request's state lives in slot seq_slot[s] of an array [slots, ...] of 32-bit
// floats and is read at the start of the request's rows and written back after its last row.  A decoded token
// is one step of the recurrence; a long portion is cut into pieces that are walked side by side (each from
// zero, then the states between the pieces, then each from its own), and lightning attention takes 32 tokens
// at a time on the matrix cores: the same sums in another order, so what a token gets depends on how the
// tokens were cut into steps by rounding only, and never on what else the step holds.  Decays, step sizes,
// exponentials, the states and all sums are 32-bit in every build; the element type stores the projections'
// outputs and is the operand type of lightning attention's products.
#include "common.cuh"

namespace ms {

// The request that row t belongs to: the last s with seq_q_start[s] <= t (starts ascend with s).
__device__ __forceinline__ int seq_of_row(int t, const int* __restrict__ seq_q_start, int S) {
    int lo = 0, hi = S - 1;
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (seq_q_start[mid] <= t) lo = mid;
        else hi = mid - 1;
    }
    return lo;
}

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

// ---- causal convolution per channel --------------------------------------------------
// out[t, c] = silu(b[c] + sum_k w[c, k] * in[t - (taps - 1 - k), c]); an input before the step's first row of the
// request comes from the state [slots, taps - 1, C] (oldest first), one before the request's start is zero there.
__global__ __launch_bounds__(256) void causal_conv_kernel(const elem_t* __restrict__ x, int ld, const float* __restrict__ w,
                                                          const float* __restrict__ b, const float* __restrict__ state,
                                                          const int* __restrict__ seq_q_start, const int* __restrict__ seq_slot,
                                                          int S, elem_t* __restrict__ out, int C, int taps) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int s = seq_of_row(t, seq_q_start, S);
    const int j = t - seq_q_start[s];
    const float* st = state + (size_t)seq_slot[s] * (taps - 1) * C;
    float acc = b ? b[c] : 0.f;
    for (int k = 0; k < taps; ++k) {
        const int back = taps - 1 - k, idx = j - back;
        const float v = idx >= 0 ? to_f32(x[(size_t)(t - back) * ld + c]) : st[(size_t)(taps - 1 + idx) * C + c];
        acc += w[(size_t)c * taps + k] * v;
    }
    out[(size_t)t * C + c] = from_f32<elem_t>(silu_f(acc));
}

// The state after the step: the last taps - 1 inputs of each request, old ones where the step brought fewer.
constexpr int MAX_TAPS = 16;
__global__ __launch_bounds__(256) void conv_state_kernel(const elem_t* __restrict__ x, int ld, float* __restrict__ state,
                                                         const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                         const int* __restrict__ seq_slot, int C, int taps) {
    const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int n = seq_q_len[s], q0 = seq_q_start[s], keep = taps - 1;
    float* st = state + (size_t)seq_slot[s] * keep * C;
    float v[MAX_TAPS];
    for (int i = 0; i < keep; ++i) {
        const int idx = n - keep + i;  // among the step's rows; negative: an older input
        v[i] = idx >= 0 ? to_f32(x[(size_t)(q0 + idx) * ld + c]) : st[(size_t)(keep + idx) * C + c];
    }
    for (int i = 0; i < keep; ++i) st[(size_t)i * C + c] = v[i];
}

// ---- step sizes ------------------------------------------------------------------------
// dt[t, c] = softplus(b[c] + sum_r wt[r, c] * low[t, r]), low = the first R columns of the rows of `dbc`; `wt` is the
// projection transposed, [R, C], so that the threads of a wave read neighbouring numbers.  A block takes DT_ROWS rows
// and 256 channels: a weight is read once for all of its rows (eight in steps of many rows, one where rows are few and
// the blocks would not fill the chip).
template <int DT_ROWS>
__global__ __launch_bounds__(256) void dt_softplus_kernel(const float* __restrict__ dbc, int ldb, const float* __restrict__ wt,
                                                          const float* __restrict__ b, float* __restrict__ dt, int T, int C, int R) {
    extern __shared__ float low[];  // [DT_ROWS][R]
    const int t0 = blockIdx.x * DT_ROWS, c = blockIdx.y * 256 + threadIdx.x;
    const int nr = min(DT_ROWS, T - t0);
    for (int i = threadIdx.x; i < nr * R; i += 256) low[i] = dbc[(size_t)(t0 + i / R) * ldb + i % R];
    __syncthreads();
    if (c >= C) return;
    float acc[DT_ROWS];
    const float bias = b ? b[c] : 0.f;
#pragma unroll
    for (int k = 0; k < DT_ROWS; ++k) acc[k] = bias;
#pragma unroll 8
    for (int r = 0; r < R; ++r) {
        const float w = wt[(size_t)r * C + c];
#pragma unroll
        for (int k = 0; k < DT_ROWS; ++k) acc[k] += w * low[(k < nr ? k : 0) * R + r];
    }
#pragma unroll
    for (int k = 0; k < DT_ROWS; ++k)
        if (k < nr) dt[(size_t)(t0 + k) * C + c] = softplus_f(acc[k]);
}

// ---- selective scan --------------------------------------------------------------------
// A channel's N states are spread over NL neighbouring lanes (NL a power of two, SPL states a lane), so a wave holds
// 64 / NL channels and a request's channels fill the chip even where one sequence is all there is.  Per token:
// S[n] = exp(dt * A[n]) * S[n] + dt * x * B[t, n];  y = sum_n S[n] * C[t, n] + D * x;  out = y * silu(z);
// the sum over the states is a reduction over the channel's lanes.
constexpr int SCAN_TILE = 16;
// A request's rows in one walk; or cut into chunks that are walked side by side: first each from zero (what it adds),
// then, after the states that come into the chunks are known (scan_carry_kernel), each from its own.
enum ScanMode { SCAN_WHOLE = 0, SCAN_LOCAL = 1, SCAN_FINAL = 2 };
template <int SPL>
__global__ __launch_bounds__(256) void selective_scan_kernel(const elem_t* __restrict__ x, const elem_t* __restrict__ z, int ldz,
                                                             const float* __restrict__ dt, const float* __restrict__ dbc, int ldb,
                                                             int col_b, int col_c, const float* __restrict__ a_log,
                                                             const float* __restrict__ dskip, float* __restrict__ state,
                                                             const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                             const int* __restrict__ seq_slot, elem_t* __restrict__ y, int C, int N, int NL,
                                                             int mode, int chunk_len, int n_chunks, float* __restrict__ carry,
                                                             float* __restrict__ csum) {
    const int s = blockIdx.x, per_block = 256 / NL;
    const int sub = threadIdx.x % NL, c = blockIdx.y * per_block + threadIdx.x / NL;
    const bool live = c < C;
    const int cc = live ? c : C - 1;
    const int q0 = seq_q_start[s] + (mode == SCAN_WHOLE ? 0 : blockIdx.z * chunk_len);
    const int left = seq_q_len[s] - (mode == SCAN_WHOLE ? 0 : blockIdx.z * chunk_len);
    if (left <= 0) return;  // the same for every thread of the block
    const int n_rows = mode == SCAN_WHOLE ? left : min(left, chunk_len);
    const bool last = n_rows == left;
    if (mode == SCAN_LOCAL && last) return;  // nobody needs what the last chunk passes on
    float* st = state + ((size_t)seq_slot[s] * C + cc) * N;
    float* pass = mode == SCAN_WHOLE ? nullptr : carry + (((size_t)s * n_chunks + blockIdx.z) * C + cc) * N;
    float S[SPL], A[SPL];
    int ns[SPL];
#pragma unroll
    for (int k = 0; k < SPL; ++k) {
        const int n = sub + k * NL;
        ns[k] = n < N ? n : -1;
        S[k] = n >= N || mode == SCAN_LOCAL ? 0.f : mode == SCAN_WHOLE ? st[n] : pass[n];
        A[k] = n < N ? -expf(a_log[(size_t)cc * N + n]) : 0.f;
    }
    float dsum = 0.f;
    const float dsk = dskip ? dskip[cc] : 0.f;
    // SCAN_TILE tokens' numbers are asked for at once, a tile ahead of the one in use: the walk is one dependent chain,
    // and a trip to memory per token would be all of its time
    struct Tile {
        float d[SCAN_TILE], xv[SCAN_TILE], zv[SCAN_TILE], Bn[SCAN_TILE][SPL], Cn[SCAN_TILE][SPL];
    };
    auto fetch = [&](int i0, Tile& tl) {
#pragma unroll
        for (int j = 0; j < SCAN_TILE; ++j) {
            const size_t t = (size_t)(q0 + min(i0 + j, n_rows - 1));
            tl.d[j] = dt[t * C + cc];
            tl.xv[j] = to_f32(x[t * C + cc]);
            tl.zv[j] = to_f32(z[t * ldz + cc]);
#pragma unroll
            for (int k = 0; k < SPL; ++k) {
                const int n = ns[k] >= 0 ? ns[k] : 0;
                tl.Bn[j][k] = dbc[t * ldb + col_b + n];
                tl.Cn[j][k] = dbc[t * ldb + col_c + n];
            }
        }
    };
    Tile cur, nxt;
    if (n_rows > 0) fetch(0, cur);
    for (int i0 = 0; i0 < n_rows; i0 += SCAN_TILE) {
        if (i0 + SCAN_TILE < n_rows) fetch(i0 + SCAN_TILE, nxt);
#pragma unroll
        for (int j = 0; j < SCAN_TILE; ++j) {
            if (i0 + j < n_rows) {  // the same for every thread of the block
                const float d = cur.d[j], xv = cur.xv[j], dx = d * xv;
                dsum += d;
                float acc = 0.f;
#pragma unroll
                for (int k = 0; k < SPL; ++k) {
                    if (ns[k] >= 0) {
#ifdef MS_ELEM_HALF
                        S[k] = __expf(d * A[k]) * S[k] + dx * cur.Bn[j][k];
#else
                        S[k] = expf(d * A[k]) * S[k] + dx * cur.Bn[j][k];
#endif
                        acc += S[k] * cur.Cn[j][k];
                    }
                }
                if (mode != SCAN_LOCAL) {  // the same for every thread
                    for (int o = NL >> 1; o > 0; o >>= 1) acc += __shfl_xor(acc, o, WAVE);
                    if (sub == 0 && live) y[(size_t)(q0 + i0 + j) * C + c] = from_f32<elem_t>((acc + dsk * xv) * silu_f(cur.zv[j]));
                }
            }
        }
        cur = nxt;
    }
    if (!live) return;
    if (mode == SCAN_LOCAL) {  // what the chunk adds to a state that comes in, and the sum of its step sizes
#pragma unroll
        for (int k = 0; k < SPL; ++k)
            if (ns[k] >= 0) pass[ns[k]] = S[k];
        if (sub == 0) csum[((size_t)s * n_chunks + blockIdx.z) * C + c] = dsum;
    } else if (mode == SCAN_WHOLE || last) {
#pragma unroll
        for (int k = 0; k < SPL; ++k)
            if (ns[k] >= 0) st[ns[k]] = S[k];
    }
}

// The chunks of a long portion are many, so there a thread takes a whole channel, its states in registers: no sum over
// lanes, and what belongs to the channel (step size, input, gate) is worked out once, not once a state.
constexpr int WIDE_TILE = 8;
template <int NMAX>
__global__ __launch_bounds__(64) void selective_scan_wide_kernel(const elem_t* __restrict__ x, const elem_t* __restrict__ z, int ldz,
                                                                 const float* __restrict__ dt, const float* __restrict__ dbc, int ldb,
                                                                 int col_b, int col_c, const float* __restrict__ a_log,
                                                                 const float* __restrict__ dskip, float* __restrict__ state,
                                                                 const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                                 const int* __restrict__ seq_slot, elem_t* __restrict__ y, int C, int N,
                                                                 int mode, int chunk_len, int n_chunks, float* __restrict__ carry,
                                                                 float* __restrict__ csum) {
    const int s = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
    const int left = seq_q_len[s] - blockIdx.z * chunk_len;
    if (left <= 0) return;
    const int q0 = seq_q_start[s] + blockIdx.z * chunk_len, n_rows = min(left, chunk_len);
    const bool last = n_rows == left;
    if ((mode == SCAN_LOCAL && last) || c >= C) return;
    float* pass = carry + (((size_t)s * n_chunks + blockIdx.z) * C + c) * N;
    float S[NMAX], A[NMAX];
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
        S[n] = (n < N && mode != SCAN_LOCAL) ? pass[n] : 0.f;
        A[n] = n < N ? -expf(a_log[(size_t)c * N + n]) : 0.f;
    }
    const float dsk = dskip ? dskip[c] : 0.f;
    float dsum = 0.f;
    for (int i0 = 0; i0 < n_rows; i0 += WIDE_TILE) {
        float d[WIDE_TILE], xv[WIDE_TILE], zv[WIDE_TILE];
#pragma unroll
        for (int j = 0; j < WIDE_TILE; ++j) {  // a tile's numbers at once
            const size_t t = (size_t)(q0 + min(i0 + j, n_rows - 1));
            d[j] = dt[t * C + c];
            xv[j] = to_f32(x[t * C + c]);
            zv[j] = mode == SCAN_LOCAL ? 0.f : to_f32(z[t * ldz + c]);
        }
#pragma unroll
        for (int j = 0; j < WIDE_TILE; ++j) {
            if (i0 + j < n_rows) {
                const float* Bt = dbc + (size_t)(q0 + i0 + j) * ldb + col_b;
                const float* Ct = dbc + (size_t)(q0 + i0 + j) * ldb + col_c;
                const float dx = d[j] * xv[j];
                dsum += d[j];
                float acc = 0.f;
#pragma unroll
                for (int n = 0; n < NMAX; ++n) {
                    if (n < N) {
#ifdef MS_ELEM_HALF
                        S[n] = __expf(d[j] * A[n]) * S[n] + dx * Bt[n];
#else
                        S[n] = expf(d[j] * A[n]) * S[n] + dx * Bt[n];
#endif
                        acc += S[n] * Ct[n];
                    }
                }
                if (mode != SCAN_LOCAL) y[(size_t)(q0 + i0 + j) * C + c] = from_f32<elem_t>((acc + dsk * xv[j]) * silu_f(zv[j]));
            }
        }
    }
    if (mode == SCAN_LOCAL) {
#pragma unroll
        for (int n = 0; n < NMAX; ++n)
            if (n < N) pass[n] = S[n];
        csum[((size_t)s * n_chunks + blockIdx.z) * C + c] = dsum;
    } else if (last) {
        float* st = state + ((size_t)seq_slot[s] * C + c) * N;
#pragma unroll
        for (int n = 0; n < NMAX; ++n)
            if (n < N) st[n] = S[n];
    }
}

// Between the two passes over the chunks: carry[s, ch] holds what chunk ch adds from zero and receives the state that
// comes into it, S_in(ch + 1) = exp(A * sum of the chunk's step sizes) * S_in(ch) + what it adds.
__global__ __launch_bounds__(256) void scan_carry_kernel(const float* __restrict__ a_log, const float* __restrict__ state,
                                                         const int* __restrict__ seq_q_len, const int* __restrict__ seq_slot,
                                                         float* __restrict__ carry, const float* __restrict__ csum, int C, int N,
                                                         int chunk_len, int n_chunks) {
    const int s = blockIdx.x;
    const size_t idx = (size_t)blockIdx.y * 256 + threadIdx.x;
    if (idx >= (size_t)C * N) return;
    const int c = (int)(idx / N);
    const int nch = (seq_q_len[s] + chunk_len - 1) / chunk_len;
    const float A = -expf(a_log[idx]);
    float Sin = state[(size_t)seq_slot[s] * C * N + idx];
    for (int ch = 0; ch < nch; ++ch) {
        float* p = carry + ((size_t)s * n_chunks + ch) * C * N + idx;
        const float add = ch + 1 < nch ? *p : 0.f;
        *p = Sin;
        if (ch + 1 < nch) Sin = expf(A * csum[((size_t)s * n_chunks + ch) * C + c]) * Sin + add;
    }
}

// ---- linear attention with a decay per head ---------------------------------------------
// qkv rows hold, before their activation, q [H, d], k [H, d], v [H, dv] at columns col_q, col_k, col_v.  A block
// is one (request, head, 64 value columns); a thread keeps column e of the head's state S [d, dv] in registers.
// Per token: S[:, e] = decay * S[:, e] + silu(k) * silu(v[e]);  o[e] = sum_d S[d, e] * silu(q[d]).  The tokens'
// q and k are activated a tile at a time into LDS, where every thread reads them.
constexpr int LIN_TILE = 16;
template <int DMAX>
__global__ __launch_bounds__(64) void lightning_kernel(const elem_t* __restrict__ qkv, int ld, int col_q, int col_k, int col_v,
                                                       const float* __restrict__ decay, float* __restrict__ state,
                                                       const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                       const int* __restrict__ seq_slot, float* __restrict__ o, int H, int d, int dv) {
    __shared__ float qs[LIN_TILE][DMAX], ks[LIN_TILE][DMAX];
    const int s = blockIdx.x, h = blockIdx.y, e = blockIdx.z * 64 + threadIdx.x;
    const bool live = e < dv;
    const int q0 = seq_q_start[s], n_rows = seq_q_len[s];
    float* st = state + (((size_t)seq_slot[s] * H + h) * d) * dv + (live ? e : 0);
    const float lam = decay[h];
    float S[DMAX];
#pragma unroll
    for (int i = 0; i < DMAX; ++i) S[i] = (live && i < d) ? st[(size_t)i * dv] : 0.f;
    for (int i0 = 0; i0 < n_rows; i0 += LIN_TILE) {
        const int nt = min(LIN_TILE, n_rows - i0);
        __syncthreads();
        for (int it = threadIdx.x; it < nt * d; it += 64) {
            const int r = it / d, c = it - r * d;
            const elem_t* row = qkv + (size_t)(q0 + i0 + r) * ld;
            qs[r][c] = silu_f(to_f32(row[col_q + h * d + c]));
            ks[r][c] = silu_f(to_f32(row[col_k + h * d + c]));
        }
        __syncthreads();
        for (int r = 0; r < nt; ++r) {
            const size_t t = (size_t)(q0 + i0 + r);
            const float v = live ? silu_f(to_f32(qkv[t * ld + col_v + h * dv + e])) : 0.f;
            float acc = 0.f;
#pragma unroll
            for (int i = 0; i < DMAX; ++i) {
                if (i < d) {
                    S[i] = lam * S[i] + ks[r][i] * v;
                    acc += S[i] * qs[r][i];
                }
            }
            if (live) o[t * ((size_t)H * dv) + (size_t)h * dv + e] = acc;
        }
    }
    if (live) {
#pragma unroll
        for (int i = 0; i < DMAX; ++i)
            if (i < d) st[(size_t)i * dv] = S[i];
    }
}

// ---- the same in chunks of 32 tokens on the matrix cores --------------------------------------
// For a chunk with tokens i, j = 0 .. n - 1 and the state S before it:
//   o_i = decay^(i + 1) S^T q_i + sum_{j <= i} decay^(i - j) (q_i . k_j) v_j,      S <- decay^n S + sum_j decay^(n - 1 - j) k_j v_j^T,
// which equals the recurrence token after token.  A block is one (request, head) and walks the request's chunks in
// order; wave w owns the value columns of the 16-wide tiles w, w + 4, ... and keeps its part of S in 32-bit
// accumulators throughout.  q, k and v are activated in 32-bit and rounded to the element type as operands of the
// products; the scores times their decays, and the state, are rounded only as operands (not at all in the 32-bit
// build), and every sum is 32-bit.
constexpr int LC = 32;  // tokens of a chunk
template <int DT, int CT>
__global__ __launch_bounds__(256) void lightning_chunk_kernel(const elem_t* __restrict__ qkv, int ld, int col_q, int col_k, int col_v,
                                                              const float* __restrict__ decay, float* __restrict__ state,
                                                              const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                              const int* __restrict__ seq_slot, float* __restrict__ o, int H, int d, int dv,
                                                              int mode, int seg_len, int n_segs, float* __restrict__ carry) {
    constexpr int DP = DT * 16, VP = CT * 64;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    elem_t* Qs = reinterpret_cast<elem_t*>(smem);  // [LC][DP]
    elem_t* Ks = Qs + LC * DP;                     // [LC][DP]
    elem_t* VT = Ks + LC * DP;                     // [VP][LC]: values transposed
    elem_t* Ps = VT + VP * LC;                     // [LC][LC]: scores times decays
    float* pw = reinterpret_cast<float*>(Ps + LC * LC);  // [LC + 1]: decay^k
    const int s = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r16 = lane & 15, grp = lane >> 4;
    // a request's rows in one walk (SCAN_WHOLE), or in segments of seg_len rows (a multiple of the chunk) that are walked
    // side by side: first each from zero, leaving what it adds (SCAN_LOCAL), then each from the state that comes into it
    const int seg0 = mode == SCAN_WHOLE ? 0 : blockIdx.z * seg_len;
    const int left = seq_q_len[s] - seg0;
    if (left <= 0) return;
    const int q0 = seq_q_start[s] + seg0, n_rows = mode == SCAN_WHOLE ? left : min(left, seg_len);
    const bool last = n_rows == left;
    if (mode == SCAN_LOCAL && last) return;
    float* st = mode == SCAN_WHOLE ? state + (((size_t)seq_slot[s] * H + h) * d) * dv
                                   : carry + ((((size_t)s * n_segs + blockIdx.z) * H + h) * d) * dv;
    const float lam = decay[h];
    if (tid <= LC) pw[tid] = powf(lam, (float)tid);
    f32x4 S[DT][CT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int e = (wave + 4 * c) * 16 + r16;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dd = dt * 16 + grp * 4 + i;
                S[dt][c][i] = (dd < d && e < dv && mode != SCAN_LOCAL) ? st[(size_t)dd * dv + e] : 0.f;
            }
        }
    const size_t orow = (size_t)H * dv;
    // a chunk's rows are asked for a chunk ahead (before their activation), so that the trip to memory runs beside the
    // chunk in work; thread tid holds elements tid, tid + 256, ... of the [LC][DP] and [LC][VP] tiles
    constexpr int QN = LC * DP / 256, VN = LC * VP / 256;
    float qn[QN], kn[QN], vn[VN];
    auto fetch = [&](int i0) {
        const int n = min(LC, n_rows - i0);
#pragma unroll
        for (int u = 0; u < QN; ++u) {
            const int idx = tid + u * 256, r = idx / DP, c = idx - r * DP;
            qn[u] = kn[u] = 0.f;
            if (r < n && c < d) {
                const elem_t* row = qkv + (size_t)(q0 + i0 + r) * ld + h * d + c;
                qn[u] = to_f32(row[col_q]);
                kn[u] = to_f32(row[col_k]);
            }
        }
#pragma unroll
        for (int u = 0; u < VN; ++u) {
            const int idx = tid + u * 256, r = idx / VP, e = idx - r * VP;
            vn[u] = (r < n && e < dv) ? to_f32(qkv[(size_t)(q0 + i0 + r) * ld + col_v + h * dv + e]) : 0.f;
        }
    };
    if (n_rows > 0) fetch(0);
    for (int i0 = 0; i0 < n_rows; i0 += LC) {
        const int n = min(LC, n_rows - i0);
        __syncthreads();  // the chunk before has been read
#pragma unroll
        for (int u = 0; u < QN; ++u) {
            const int idx = tid + u * 256;
            Qs[idx] = from_f32<elem_t>(silu_f(qn[u]));   // silu(0) = 0: what lies beyond the rows and the head stays zero
            Ks[idx] = from_f32<elem_t>(silu_f(kn[u]));
        }
#pragma unroll
        for (int u = 0; u < VN; ++u) {
            const int idx = tid + u * 256, r = idx / VP, e = idx - r * VP;
            VT[e * LC + r] = from_f32<elem_t>(silu_f(vn[u]));
        }
        if (i0 + LC < n_rows) fetch(i0 + LC);
        __syncthreads();
        {   // a quarter of the scores a wave: rows rt, columns ct
            const int rt = wave >> 1, ct = wave & 1;
            f32x4 p = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < DT / 2; ++ks) {
                const Frag qa = frag_load(&Qs[(rt * 16 + r16) * DP + ks * 32 + grp * 8]);
                const Frag kb = frag_load(&Ks[(ct * 16 + r16) * DP + ks * 32 + grp * 8]);
                mma_16x16x32(p, qa, kb);
            }
            const int j = ct * 16 + r16;
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) {
                const int i = rt * 16 + grp * 4 + ii;
                Ps[i * LC + j] = from_f32<elem_t>(j <= i ? p[ii] * pw[i - j] : 0.f);
            }
        }
        // what the state before the chunk gives: rows are tokens, the sum runs over the head's numbers in pairs of tiles
        f32x4 O[2][CT];
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int c = 0; c < CT; ++c) O[rt][c] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t2 = 0; t2 < DT / 2; ++t2) {
            Frag qa[2];
#pragma unroll
            for (int rt = 0; rt < 2; ++rt) {
                const elem_t* qp = &Qs[(rt * 16 + r16) * DP + t2 * 32 + grp * 4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    qa[rt].v[i] = qp[i];
                    qa[rt].v[4 + i] = qp[16 + i];
                }
            }
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                Frag sb;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    sb.v[i] = from_f32<elem_t>(S[2 * t2][c][i]);
                    sb.v[4 + i] = from_f32<elem_t>(S[2 * t2 + 1][c][i]);
                }
#pragma unroll
                for (int rt = 0; rt < 2; ++rt) mma_16x16x32(O[rt][c], qa[rt], sb);
            }
        }
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int ii = 0; ii < 4; ++ii) {
                const float f = pw[rt * 16 + grp * 4 + ii + 1];
#pragma unroll
                for (int c = 0; c < CT; ++c) O[rt][c][ii] *= f;
            }
        __syncthreads();  // the scores are complete
        Frag vb[CT];
#pragma unroll
        for (int c = 0; c < CT; ++c) vb[c] = frag_load(&VT[((wave + 4 * c) * 16 + r16) * LC + grp * 8]);
#pragma unroll
        for (int rt = 0; rt < 2; ++rt) {
            const Frag pa = frag_load(&Ps[(rt * 16 + r16) * LC + grp * 8]);
#pragma unroll
            for (int c = 0; c < CT; ++c) mma_16x16x32(O[rt][c], pa, vb[c]);
        }
#pragma unroll
        for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                const int e = (wave + 4 * c) * 16 + r16;
#pragma unroll
                for (int ii = 0; ii < 4; ++ii) {
                    const int i = rt * 16 + grp * 4 + ii;
                    if (i < n && e < dv && mode != SCAN_LOCAL) o[(size_t)(q0 + i0 + i) * orow + (size_t)h * dv + e] = O[rt][c][ii];
                }
            }
        // the state after the chunk
        const float ln = pw[n];
        float kw[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int j = grp * 8 + i;
            kw[i] = j < n ? pw[n - 1 - j] : 0.f;
        }
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
            Frag ka;
#pragma unroll
            for (int i = 0; i < 8; ++i) ka.v[i] = from_f32<elem_t>(to_f32(Ks[(grp * 8 + i) * DP + dt * 16 + r16]) * kw[i]);
#pragma unroll
            for (int c = 0; c < CT; ++c) {
                S[dt][c] *= ln;
                mma_16x16x32(S[dt][c], ka, vb[c]);
            }
        }
    }
    // the state after the rows: into the workspace what a segment adds; into the request's slot after its last row
    float* dst = mode == SCAN_LOCAL ? st : (mode == SCAN_WHOLE || last) ? state + (((size_t)seq_slot[s] * H + h) * d) * dv : nullptr;
    if (dst == nullptr) return;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int c = 0; c < CT; ++c) {
            const int e = (wave + 4 * c) * 16 + r16;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int dd = dt * 16 + grp * 4 + i;
                if (dd < d && e < dv) dst[(size_t)dd * dv + e] = S[dt][c][i];
            }
        }
}

// Between the two passes over the segments: carry[s, g, h] holds what segment g adds from zero and receives the state
// that comes into it, S_in(g + 1) = decay^(rows of g) * S_in(g) + what g adds.
__global__ __launch_bounds__(256) void lightning_carry_kernel(const float* __restrict__ decay, const float* __restrict__ state,
                                                              const int* __restrict__ seq_q_len, const int* __restrict__ seq_slot,
                                                              float* __restrict__ carry, int H, int per_head, int seg_len, int n_segs) {
    const int s = blockIdx.x, h = blockIdx.y, i = blockIdx.z * 256 + threadIdx.x;
    if (i >= per_head) return;
    const int n = seq_q_len[s], segs = (n + seg_len - 1) / seg_len;
    const float f = powf(decay[h], (float)seg_len);  // every segment that passes something on is a whole one
    float Sin = state[((size_t)seq_slot[s] * H + h) * per_head + i];
    for (int g = 0; g < segs; ++g) {
        float* p = carry + (((size_t)s * n_segs + g) * H + h) * per_head + i;
        const float add = g + 1 < segs ? *p : 0.f;
        *p = Sin;
        if (g + 1 < segs) Sin = f * Sin + add;
    }
}

// out[t, :] = o[t, :] / sqrt(mean(o[t, :]^2) + eps) * w * sigmoid(gate[t, :])
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const float* __restrict__ o, const elem_t* __restrict__ gate, int ldg,
                                                            const float* __restrict__ w, elem_t* __restrict__ out, int n, float eps) {
    __shared__ float scratch[4];
    const int t = blockIdx.x;
    const float* row = o + (size_t)t * n;
    float ss = 0.f;
    for (int c = threadIdx.x; c < n; c += 256) ss += row[c] * row[c];
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)n + eps);
    for (int c = threadIdx.x; c < n; c += 256)
        out[(size_t)t * n + c] = from_f32<elem_t>(row[c] * inv * w[c] * sigmoid_f(to_f32(gate[(size_t)t * ldg + c])));
}

}  // namespace ms

using namespace ms;

extern "C" int ms_conv_max_taps() { return MAX_TAPS; }
extern "C" int ms_scan_max_states() { return 128; }
extern "C" int ms_lightning_max_dim() { return 256; }

// x: the convolution's input, column c of rows of stride ld; state float [slots, taps - 1, C]; out [T, C].
extern "C" int ms_causal_conv(const void* x, int ld, const float* w, const float* b, float* state, const int* seq_q_start,
                              const int* seq_q_len, const int* seq_slot, int S, void* out, int T, int C, int taps,
                              hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && C > 0 && ld >= C, "causal convolution: T=%d S=%d C=%d ld=%d", T, S, C, ld);
    MS_REQUIRE(taps >= 1 && taps <= MAX_TAPS, "causal convolution: %d taps, at most %d are built", taps, MAX_TAPS);
    MS_REQUIRE(x && w && state && seq_q_start && seq_q_len && seq_slot && out, "causal convolution: a buffer is missing");
    const unsigned cb = (unsigned)ceil_div(C, 256);
    hipLaunchKernelGGL(causal_conv_kernel, dim3(T, cb), dim3(256), 0, stream, (const elem_t*)x, ld, w, b, state, seq_q_start,
                       seq_slot, S, (elem_t*)out, C, taps);
    if (int rc = check_launch("causal convolution")) return rc;
    if (taps > 1) {
        hipLaunchKernelGGL(conv_state_kernel, dim3(S, cb), dim3(256), 0, stream, (const elem_t*)x, ld, state, seq_q_start,
                           seq_q_len, seq_slot, C, taps);
        return check_launch("causal convolution state");
    }
    return 0;
}

// w: the projection of the step sizes transposed, [R, C]
extern "C" int ms_dt_softplus(const float* dbc, int ldb, const float* w, const float* b, float* dt, int T, int C, int R,
                              hipStream_t stream) {
    MS_REQUIRE(T > 0 && C > 0 && R > 0 && ldb >= R, "step sizes: T=%d C=%d R=%d ld=%d", T, C, R, ldb);
    MS_REQUIRE(dbc && w && dt, "step sizes: a buffer is missing");
    MS_REQUIRE((size_t)8 * R * sizeof(float) <= 48 * 1024, "step sizes: a bottleneck of %d is too wide", R);
    if (T >= 128)
        hipLaunchKernelGGL(dt_softplus_kernel<8>, dim3(ceil_div(T, 8), ceil_div(C, 256)), dim3(256), (size_t)8 * R * sizeof(float), stream, dbc,
                           ldb, w, b, dt, T, C, R);
    else
        hipLaunchKernelGGL(dt_softplus_kernel<1>, dim3(T, ceil_div(C, 256)), dim3(256), (size_t)R * sizeof(float), stream, dbc, ldb, w, b, dt,
                           T, C, R);
    return check_launch("step sizes");
}

extern "C" int ms_selective_scan(const void* x, const void* z, int ldz, const float* dt, const float* dbc, int ldb, int col_b,
                                 int col_c, const float* a_log, const float* dskip, float* state, const int* seq_q_start,
                                 const int* seq_q_len, const int* seq_slot, int S, void* y, int T, int C, int N, int chunk_len,
                                 int n_chunks, float* carry, float* csum, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && C > 0 && N > 0, "selective scan: T=%d S=%d C=%d N=%d", T, S, C, N);
    MS_REQUIRE(N <= 128, "selective scan: %d states a channel, at most 128 are built", N);
    MS_REQUIRE(col_b >= 0 && col_c >= 0 && col_b + N <= ldb && col_c + N <= ldb, "selective scan: columns %d, %d of rows of %d", col_b, col_c, ldb);
    MS_REQUIRE(x && z && dt && dbc && a_log && state && seq_q_start && seq_q_len && seq_slot && y, "selective scan: a buffer is missing");
    MS_REQUIRE(chunk_len == 0 || (chunk_len > 0 && n_chunks > 0 && carry && csum), "selective scan: chunks of %d need their workspace", chunk_len);
    int nl = 1;
    while (nl < N && nl < 64) nl *= 2;
#define MS_SCAN(SP, MODE, Z)                                                                                                       \
    hipLaunchKernelGGL(selective_scan_kernel<SP>, dim3(S, ceil_div(C, 256 / nl), Z), dim3(256), 0, stream, (const elem_t*)x,          \
                       (const elem_t*)z, ldz, dt, dbc, ldb, col_b, col_c, a_log, dskip, state, seq_q_start, seq_q_len, seq_slot,     \
                       (elem_t*)y, C, N, nl, MODE, chunk_len, n_chunks, carry, csum)
#define MS_SCAN_N(MODE, Z)            \
    do {                              \
        if (N <= 64) MS_SCAN(1, MODE, Z); \
        else MS_SCAN(2, MODE, Z);     \
    } while (0)
    if (chunk_len == 0) {
        MS_SCAN_N(SCAN_WHOLE, 1);
    } else if (N <= 32) {  // a channel a thread, its states in registers
#define MS_WIDE(NM, MODE)                                                                                                          \
    hipLaunchKernelGGL(selective_scan_wide_kernel<NM>, dim3(S, ceil_div(C, 64), n_chunks), dim3(64), 0, stream, (const elem_t*)x,    \
                       (const elem_t*)z, ldz, dt, dbc, ldb, col_b, col_c, a_log, dskip, state, seq_q_start, seq_q_len, seq_slot,     \
                       (elem_t*)y, C, N, MODE, chunk_len, n_chunks, carry, csum)
        if (N <= 16) MS_WIDE(16, SCAN_LOCAL);
        else MS_WIDE(32, SCAN_LOCAL);
        if (int rc = check_launch("selective scan, chunks from zero")) return rc;
        hipLaunchKernelGGL(scan_carry_kernel, dim3(S, (unsigned)ceil_div((long)C * N, 256L)), dim3(256), 0, stream, a_log, state, seq_q_len,
                           seq_slot, carry, csum, C, N, chunk_len, n_chunks);
        if (int rc = check_launch("selective scan, states between chunks")) return rc;
        if (N <= 16) MS_WIDE(16, SCAN_FINAL);
        else MS_WIDE(32, SCAN_FINAL);
#undef MS_WIDE
    } else {
        MS_SCAN_N(SCAN_LOCAL, n_chunks);
        if (int rc = check_launch("selective scan, chunks from zero")) return rc;
        hipLaunchKernelGGL(scan_carry_kernel, dim3(S, (unsigned)ceil_div((long)C * N, 256L)), dim3(256), 0, stream, a_log, state, seq_q_len,
                           seq_slot, carry, csum, C, N, chunk_len, n_chunks);
        if (int rc = check_launch("selective scan, states between chunks")) return rc;
        MS_SCAN_N(SCAN_FINAL, n_chunks);
    }
#undef MS_SCAN_N
#undef MS_SCAN
    return check_launch("selective scan");
}

extern "C" int ms_lightning(const void* qkv, int ld, int col_q, int col_k, int col_v, const float* decay, float* state,
                            const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, float* o, int T, int H,
                            int d, int dv, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && H > 0 && d > 0 && dv > 0, "lightning attention: T=%d S=%d H=%d d=%d dv=%d", T, S, H, d, dv);
    MS_REQUIRE(d <= 256, "lightning attention: heads of %d, at most 256 are built", d);
    MS_REQUIRE(col_q >= 0 && col_k >= 0 && col_v >= 0 && col_q + H * d <= ld && col_k + H * d <= ld && col_v + H * dv <= ld,
               "lightning attention: columns %d, %d, %d of rows of %d", col_q, col_k, col_v, ld);
    MS_REQUIRE(qkv && decay && state && seq_q_start && seq_q_len && seq_slot && o, "lightning attention: a buffer is missing");
    const dim3 grid(S, H, ceil_div(dv, 64));
#define MS_LIN(DM)                                                                                                         \
    hipLaunchKernelGGL(lightning_kernel<DM>, grid, dim3(64), 0, stream, (const elem_t*)qkv, ld, col_q, col_k, col_v, decay, \
                       state, seq_q_start, seq_q_len, seq_slot, o, H, d, dv)
    if (d <= 32) MS_LIN(32);
    else if (d <= 64) MS_LIN(64);
    else if (d <= 128) MS_LIN(128);
    else MS_LIN(256);
#undef MS_LIN
    return check_launch("lightning attention");
}

extern "C" int ms_gated_rmsnorm(const float* o, const void* gate, int ldg, const float* w, void* out, int T, int n, float eps,
                                hipStream_t stream) {
    MS_REQUIRE(T > 0 && n > 0 && ldg >= n, "gated norm: T=%d n=%d ld=%d", T, n, ldg);
    MS_REQUIRE(o && gate && w && out, "gated norm: a buffer is missing");
    hipLaunchKernelGGL(gated_rmsnorm_kernel, dim3(T), dim3(256), 0, stream, o, (const elem_t*)gate, ldg, w, (elem_t*)out, n, eps);
    return check_launch("gated norm");
}

// Whether the kernel that walks a request in chunks on the matrix cores takes these head sizes.
extern "C" int ms_lightning_chunked_takes(int d, int dv) { return d >= 1 && d <= 128 && dv >= 1 && dv <= 128; }

// seg_len > 0 (a multiple of 32): the requests' rows in segments walked side by side, with carry float
// [S, n_segs, H, d, dv] as workspace; 0: each request in one walk.
extern "C" int ms_lightning_chunked(const void* qkv, int ld, int col_q, int col_k, int col_v, const float* decay, float* state,
                                    const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, float* o, int T, int H,
                                    int d, int dv, int seg_len, int n_segs, float* carry, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && H > 0, "lightning attention: T=%d S=%d H=%d", T, S, H);
    MS_REQUIRE(ms_lightning_chunked_takes(d, dv), "lightning attention in chunks: heads of %d and values of %d are not taken", d, dv);
    MS_REQUIRE(col_q >= 0 && col_k >= 0 && col_v >= 0 && col_q + H * d <= ld && col_k + H * d <= ld && col_v + H * dv <= ld,
               "lightning attention: columns %d, %d, %d of rows of %d", col_q, col_k, col_v, ld);
    MS_REQUIRE(qkv && decay && state && seq_q_start && seq_q_len && seq_slot && o, "lightning attention: a buffer is missing");
    MS_REQUIRE(seg_len == 0 || (seg_len % LC == 0 && n_segs > 0 && carry), "lightning attention in chunks: segments of %d need their workspace", seg_len);
    const int dtl = d <= 32 ? 2 : d <= 64 ? 4 : 8, ctl = dv <= 64 ? 1 : 2;
#define MS_LCH(DTT, CTT, MODE, Z)                                                                                                   \
    hipLaunchKernelGGL((lightning_chunk_kernel<DTT, CTT>), dim3(S, H, Z), dim3(256),                                                 \
                       sizeof(elem_t) * (2 * LC * DTT * 16 + CTT * 64 * LC + LC * LC) + sizeof(float) * (LC + 1 + 3), stream,       \
                       (const elem_t*)qkv, ld, col_q, col_k, col_v, decay, state, seq_q_start, seq_q_len, seq_slot, o, H, d, dv, MODE, \
                       seg_len, n_segs, carry)
#define MS_LCH_ALL(MODE, Z)                                  \
    do {                                                     \
        if (dtl == 2 && ctl == 1) MS_LCH(2, 1, MODE, Z);     \
        else if (dtl == 2) MS_LCH(2, 2, MODE, Z);            \
        else if (dtl == 4 && ctl == 1) MS_LCH(4, 1, MODE, Z); \
        else if (dtl == 4) MS_LCH(4, 2, MODE, Z);            \
        else if (ctl == 1) MS_LCH(8, 1, MODE, Z);            \
        else MS_LCH(8, 2, MODE, Z);                          \
    } while (0)
    if (seg_len == 0) {
        MS_LCH_ALL(SCAN_WHOLE, 1);
    } else {
        MS_LCH_ALL(SCAN_LOCAL, n_segs);
        if (int rc = check_launch("lightning attention, segments from zero")) return rc;
        hipLaunchKernelGGL(lightning_carry_kernel, dim3(S, H, ceil_div(d * dv, 256)), dim3(256), 0, stream, decay, state, seq_q_len, seq_slot,
                           carry, H, d * dv, seg_len, n_segs);
        if (int rc = check_launch("lightning attention, states between segments")) return rc;
        MS_LCH_ALL(SCAN_FINAL, n_segs);
    }
#undef MS_LCH_ALL
#undef MS_LCH
    return check_launch("lightning attention in chunks");
}
