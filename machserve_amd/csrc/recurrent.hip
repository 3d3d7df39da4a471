// Mixers whose memory is a state of fixed size per request: the short causal convolution and the selective
// scan of a Mamba layer, and linear attention with a decay per head ("lightning" attention), with the gated
// norm that follows it.
//
// A step's rows are the tokens of several requests, each request's rows contiguous and in order
// (seq_q_start, seq_q_len); a request's state lives in slot seq_slot[s] of an array [slots, ...] of 32-bit
// floats and is read at the start of the request's rows and written back after its last row.  Every request
// is walked token after token in one fixed order, so what a token gets does not depend on how the tokens were
// cut into steps or on what else the step holds.  Decays, step sizes, exponentials and the states themselves
// are 32-bit in every build; the element type only stores the projections' outputs.
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
// dt[t, c] = softplus(b[c] + sum_r w[c, r] * low[t, r]), low = the first R columns of the rows of `dbc`
__global__ __launch_bounds__(256) void dt_softplus_kernel(const float* __restrict__ dbc, int ldb, const float* __restrict__ w,
                                                          const float* __restrict__ b, float* __restrict__ dt, int C, int R) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const float* low = dbc + (size_t)t * ldb;
    float acc = b ? b[c] : 0.f;
    for (int r = 0; r < R; ++r) acc += w[(size_t)c * R + r] * low[r];
    dt[(size_t)t * C + c] = softplus_f(acc);
}

// ---- selective scan --------------------------------------------------------------------
// One thread per (request, channel) with the channel's N states in registers.  Per token:
// S[n] = exp(dt * A[n]) * S[n] + dt * x * B[t, n];  y = sum_n S[n] * C[t, n] + D * x;  out = y * silu(z).
template <int NMAX>
__global__ __launch_bounds__(64) void selective_scan_kernel(const elem_t* __restrict__ x, const elem_t* __restrict__ z, int ldz,
                                                            const float* __restrict__ dt, const float* __restrict__ dbc, int ldb,
                                                            int col_b, int col_c, const float* __restrict__ a_log,
                                                            const float* __restrict__ dskip, float* __restrict__ state,
                                                            const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                            const int* __restrict__ seq_slot, elem_t* __restrict__ y, int C, int N) {
    const int s = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x;
    if (c >= C) return;
    const int q0 = seq_q_start[s], n_rows = seq_q_len[s];
    float* st = state + ((size_t)seq_slot[s] * C + c) * N;
    float S[NMAX], A[NMAX];
#pragma unroll
    for (int n = 0; n < NMAX; ++n) {
        S[n] = n < N ? st[n] : 0.f;
        A[n] = n < N ? -expf(a_log[(size_t)c * N + n]) : 0.f;
    }
    const float dsk = dskip ? dskip[c] : 0.f;
    for (int i = 0; i < n_rows; ++i) {
        const size_t t = (size_t)(q0 + i);
        const float d = dt[t * C + c], xv = to_f32(x[t * C + c]), zv = to_f32(z[t * ldz + c]);
        const float* Bt = dbc + t * ldb + col_b;
        const float* Ct = dbc + t * ldb + col_c;
        const float dx = d * xv;
        float acc = 0.f;
#pragma unroll
        for (int n = 0; n < NMAX; ++n) {
            if (n < N) {
                S[n] = expf(d * A[n]) * S[n] + dx * Bt[n];
                acc += S[n] * Ct[n];
            }
        }
        y[t * C + c] = from_f32<elem_t>((acc + dsk * xv) * silu_f(zv));
    }
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
        if (n < N) st[n] = S[n];
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

extern "C" int ms_dt_softplus(const float* dbc, int ldb, const float* w, const float* b, float* dt, int T, int C, int R,
                              hipStream_t stream) {
    MS_REQUIRE(T > 0 && C > 0 && R > 0 && ldb >= R, "step sizes: T=%d C=%d R=%d ld=%d", T, C, R, ldb);
    MS_REQUIRE(dbc && w && dt, "step sizes: a buffer is missing");
    hipLaunchKernelGGL(dt_softplus_kernel, dim3(T, ceil_div(C, 256)), dim3(256), 0, stream, dbc, ldb, w, b, dt, C, R);
    return check_launch("step sizes");
}

extern "C" int ms_selective_scan(const void* x, const void* z, int ldz, const float* dt, const float* dbc, int ldb, int col_b,
                                 int col_c, const float* a_log, const float* dskip, float* state, const int* seq_q_start,
                                 const int* seq_q_len, const int* seq_slot, int S, void* y, int T, int C, int N,
                                 hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && C > 0 && N > 0, "selective scan: T=%d S=%d C=%d N=%d", T, S, C, N);
    MS_REQUIRE(N <= 128, "selective scan: %d states a channel, at most 128 are built", N);
    MS_REQUIRE(col_b >= 0 && col_c >= 0 && col_b + N <= ldb && col_c + N <= ldb, "selective scan: columns %d, %d of rows of %d", col_b, col_c, ldb);
    MS_REQUIRE(x && z && dt && dbc && a_log && state && seq_q_start && seq_q_len && seq_slot && y, "selective scan: a buffer is missing");
    const dim3 grid(S, ceil_div(C, 64));
#define MS_SCAN(NM)                                                                                                          \
    hipLaunchKernelGGL(selective_scan_kernel<NM>, grid, dim3(64), 0, stream, (const elem_t*)x, (const elem_t*)z, ldz, dt, dbc, \
                       ldb, col_b, col_c, a_log, dskip, state, seq_q_start, seq_q_len, seq_slot, (elem_t*)y, C, N)
    if (N <= 16) MS_SCAN(16);
    else if (N <= 32) MS_SCAN(32);
    else if (N <= 64) MS_SCAN(64);
    else MS_SCAN(128);
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
