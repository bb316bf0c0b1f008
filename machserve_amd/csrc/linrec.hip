// Linear recurrences with gates that depend on the token, and what surrounds them: a short causal convolution over
// 32-bit sums with a state, the real-gated linear recurrent unit (gates from block-diagonal maps of the convolved
// input, S <- a S + sqrt(1 - a^2) (i * u) with a = exp(-c r softplus(lam))), the mix of a token with the one before
// it, and time mixing with a decay per key channel and token (S <- diag(w) S + k v^T, read with a bonus for the
// current token), whose heads are divided by their root mean square, weighted and gated in the same kernel.
//
// A step's rows are the tokens of several requests, each request's rows contiguous and in order (seq_q_start,
// seq_q_len); a request's state lives in slot seq_slot[s] of arrays [slots, ...] of 32-bit floats, is read at the start
// of the request's rows and written back after its last.  Gates, decays and their logarithms, exponentials, the states
// and every sum are 32-bit in every build; the element type stores what the next matrix product reads.  A row's result
// depends on its own request alone.  Short steps walk a request's rows token after token; long portions are walked in
// segments side by side whose incoming states a carry kernel chains, so that cuts of a prompt differ by that chain's
// 32-bit rounding and by nothing else.
#include "common.cuh"
#include <type_traits>

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

__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.0f ? z : log1pf(expf(z)); }
__device__ __forceinline__ float gelu_tanh_f(float z) { return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))); }

constexpr int MAX_TAPS = 16;

// ---- causal convolution over 32-bit sums -------------------------------------------------
// u[t, c] = bias_in[c] + sum_p in[p, t, col0 + c]: a projection's output, given as partial sums;
// out[t, c] = bias_out[c] + sum_k w[c, k] * u[t - (taps - 1 - k), c].  An input before the step's first row of the
// request comes from state [slots, taps - 1, C] (oldest first), which holds zeros before the request's start.
struct ConvArgs {
    const float* in;
    int n_partials;
    size_t partial_stride;
    int ld, col0;
    const float* bias_in;   // [C] or null
    const float* w;         // [C, taps]
    const float* bias_out;  // [C] or null
    float* state;           // [slots, taps - 1, C]
    const int* seq_q_start;
    const int* seq_q_len;
    const int* seq_slot;
    int S;
    float* out;             // [T, ld_out], columns out0 onwards
    int ld_out, out0;
    int C, taps;
};

__device__ __forceinline__ float conv_input(const ConvArgs& a, int t, int c) {
    float v = a.bias_in ? a.bias_in[c] : 0.f;
    const float* src = a.in + (size_t)t * a.ld + a.col0 + c;
    for (int p = 0; p < a.n_partials; ++p) v += src[p * a.partial_stride];
    return v;
}

__global__ __launch_bounds__(256) void conv_rows_kernel(ConvArgs a) {
    const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int s = seq_of_row(t, a.seq_q_start, a.S);
    const int j = t - a.seq_q_start[s];
    const int keep = a.taps - 1;
    const float* st = a.state + (size_t)a.seq_slot[s] * keep * a.C;
    float acc = a.bias_out ? a.bias_out[c] : 0.f;
    // a tap reads the step's rows or the state (which of the two is the same for the whole block); the address is chosen,
    // not the load: every load goes out on one straight path
    const float bias = a.bias_in ? a.bias_in[c] : 0.f;
#pragma unroll 4
    for (int k = 0; k < a.taps; ++k) {
        const int back = keep - k, idx = j - back;
        const bool fresh = idx >= 0;
        const float* src = fresh ? a.in + (size_t)(t - back) * a.ld + a.col0 + c : st + (size_t)(keep + idx) * a.C + c;
        const size_t stride = fresh ? a.partial_stride : 0;
        float v = fresh ? bias : 0.f;
        for (int p = 0; p < a.n_partials; ++p) {
            const float part = src[p * stride];
            v += (fresh || p == 0) ? part : 0.f;
        }
        acc += a.w[(size_t)c * a.taps + k] * v;
    }
    a.out[(size_t)t * a.ld_out + a.out0 + c] = acc;
}

// The state after the step: the last taps - 1 inputs of each request, old ones where the step brought fewer.
__global__ __launch_bounds__(256) void conv_rows_state_kernel(ConvArgs a) {
    const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= a.C) return;
    const int n = a.seq_q_len[s], q0 = a.seq_q_start[s], keep = a.taps - 1;
    float* st = a.state + (size_t)a.seq_slot[s] * keep * a.C;
    float v[MAX_TAPS];
    for (int i = 0; i < keep; ++i) {
        const int idx = n - keep + i;  // among the step's rows; negative: an older input
        v[i] = idx >= 0 ? conv_input(a, q0 + idx, c) : st[(size_t)(keep + idx) * a.C + c];
    }
    for (int i = 0; i < keep; ++i) st[(size_t)i * a.C + c] = v[i];
}

// ---- the gated linear recurrent unit ------------------------------------------------------
// Gates: the channels are cut into B blocks of bw; r = sigmoid(Wa[b] u_b + ba), i = sigmoid(Wi[b] u_b + bi);
// log a = -c r softplus(lam);  a = exp(log a);  drive = sqrt(1 - a^2) * i * u.  The weights come transposed,
// [B, bw (in), bw (out)], so that the threads of a wave, which are outputs, read neighbouring numbers.  A block of
// threads takes GATE_ROWS rows and GATE_OUTS outputs of one block of channels; its four waves each sum over a quarter
// of the inputs (a short chain of loads also where the rows are few), and the quarters meet in LDS.
constexpr int GATE_ROWS = 16, GATE_OUTS = 64, GATE_SLICES = 4;
struct GateArgs {
    const float* u;        // [T, C]
    const elem_t* wa_t;    // [B, bw, bw] transposed
    const elem_t* wi_t;
    const float* ba;       // [C]
    const float* bi;       // [C]
    const float* lam;      // [C]
    float c;               // the factor in the decay's exponent
    float* a_out;          // [T, C]
    float* drive_out;      // [T, C]
    int T, C, bw;
};

constexpr int GATE_K = 32;  // inputs whose weights a thread asks for at once

__global__ __launch_bounds__(256) void lru_gates_kernel(GateArgs g) {
    extern __shared__ __align__(16) float us[];  // [GATE_ROWS][ldu], a row's end filled with zeros
    __shared__ float part[2][GATE_SLICES][GATE_ROWS][GATE_OUTS];
    const int t0 = blockIdx.x * GATE_ROWS, b = blockIdx.y, bw = g.bw;
    const int ldu = (bw + 3) & ~3;
    const int nr = min(GATE_ROWS, g.T - t0);
    for (int i = threadIdx.x; i < GATE_ROWS * ldu; i += 256) {
        const int r = i / ldu, k = i - r * ldu;
        us[i] = (r < nr && k < bw) ? g.u[(size_t)(t0 + r) * g.C + b * bw + k] : 0.f;
    }
    const int lane = threadIdx.x & (GATE_OUTS - 1), slice = threadIdx.x / GATE_OUTS;
    const int o = blockIdx.z * GATE_OUTS + lane;
    const bool live = o < bw;
    const elem_t* wa = g.wa_t + (size_t)b * bw * bw + (live ? o : 0);
    const elem_t* wi = g.wi_t + (size_t)b * bw * bw + (live ? o : 0);
    const int per = (((bw + GATE_SLICES - 1) / GATE_SLICES) + 3) & ~3;  // a slice's inputs, whole groups of four
    const int k0 = slice * per, k1 = min(ldu, k0 + per);
    float ar[GATE_ROWS], ai[GATE_ROWS];
#pragma unroll
    for (int r = 0; r < GATE_ROWS; ++r) ar[r] = ai[r] = 0.f;
    for (int kc = k0; kc < k1; kc += GATE_K) {
        float fa[GATE_K], fi[GATE_K];
#pragma unroll
        for (int q = 0; q < GATE_K; ++q) {  // the weights of GATE_K inputs in one trip to memory
            const int k = kc + q;
            const bool in = k < k1 && k < bw;
            const size_t at = (size_t)min(k, bw - 1) * bw;  // every load goes out, on one straight path
            const float va = to_f32(wa[at]), vi = to_f32(wi[at]);
            fa[q] = in ? va : 0.f;
            fi[q] = in ? vi : 0.f;
        }
        if (kc == k0) __syncthreads();  // the rows are in LDS (the first weights were asked for meanwhile)
#pragma unroll
        for (int q = 0; q < GATE_K; q += 4) {
            if (kc + q < k1) {
#pragma unroll
                for (int r = 0; r < GATE_ROWS; ++r) {
                    const float4 u4 = *reinterpret_cast<const float4*>(&us[r * ldu + kc + q]);
                    ar[r] += fa[q] * u4.x + fa[q + 1] * u4.y + fa[q + 2] * u4.z + fa[q + 3] * u4.w;
                    ai[r] += fi[q] * u4.x + fi[q + 1] * u4.y + fi[q + 2] * u4.z + fi[q + 3] * u4.w;
                }
            }
        }
    }
    if (k0 >= k1) __syncthreads();  // a slice without inputs has not met the others yet
#pragma unroll
    for (int r = 0; r < GATE_ROWS; ++r) {
        part[0][slice][r][lane] = ar[r];
        part[1][slice][r][lane] = ai[r];
    }
    __syncthreads();
    if (!live) return;
    const int c = b * bw + o;
    const float sp = softplus_f(g.lam[c]), ba = g.ba[c], bi = g.bi[c];
    // a wave finishes a quarter of the rows; the quarters of the inputs are added in the same order for every row
    for (int r = slice; r < nr; r += GATE_SLICES) {
        float za = 0.f, zi = 0.f;
#pragma unroll
        for (int q = 0; q < GATE_SLICES; ++q) {
            za += part[0][q][r][lane];
            zi += part[1][q][r][lane];
        }
        const float rg = sigmoid_f(za + ba), ig = sigmoid_f(zi + bi);
        const float log_a = -g.c * rg * sp;
        const float av = expf(log_a);
        // 1 - a^2 = -expm1(2 log a): no cancellation where a is close to one
        const float drive = sqrtf(-expm1f(2.0f * log_a)) * ig * us[r * ldu + o];
        g.a_out[(size_t)(t0 + r) * g.C + c] = av;
        g.drive_out[(size_t)(t0 + r) * g.C + c] = drive;
    }
}

// A request's rows in one walk (WALK_WHOLE); or cut into segments that are walked side by side: first each from zero
// (WALK_LOCAL: what the segment adds, and the product of its decays), then, after the states that come into the segments
// are known (the carry kernels), each from its own (WALK_FINAL).  Within a segment the walk is token after token.
enum { WALK_WHOLE = 0, WALK_LOCAL = 1, WALK_FINAL = 2 };

// The recurrence, a channel a thread: S <- a S + drive;  out = S * gelu_tanh(y + by), with y the other branch's projection
// in the element type (columns ycol onwards of rows of ld elements).  carry [S, n_segs, 2, C]: the product of a segment's
// decays and what it adds; the first of the two is replaced by the state that comes into the segment.
constexpr int LRU_AHEAD = 8;
template <int MODE>
__global__ __launch_bounds__(64) void lru_scan_kernel(const float* __restrict__ a, const float* __restrict__ drive,
                                                      const elem_t* __restrict__ y, int ldy, int ycol, const float* __restrict__ by,
                                                      float* __restrict__ state, const int* __restrict__ seq_q_start,
                                                      const int* __restrict__ seq_q_len, const int* __restrict__ seq_slot,
                                                      elem_t* __restrict__ out, int C, int seg_len, int n_segs,
                                                      float* __restrict__ carry) {
    const int s = blockIdx.x, c = blockIdx.y * 64 + threadIdx.x, seg = blockIdx.z;
    if (c >= C) return;
    const int off = MODE == WALK_WHOLE ? 0 : seg * seg_len;
    const int left = seq_q_len[s] - off;
    if (left <= 0) return;
    const int n = MODE == WALK_WHOLE ? left : min(left, seg_len);
    const bool last = MODE == WALK_WHOLE || left <= seg_len;
    if (MODE == WALK_LOCAL && last) return;  // nobody needs what the last segment passes on
    const int q0 = seq_q_start[s] + off;
    float* st = state + (size_t)seq_slot[s] * C + c;
    float* pass = MODE == WALK_WHOLE ? nullptr : carry + ((size_t)s * n_segs + seg) * 2 * C + c;
    float S = MODE == WALK_WHOLE ? *st : MODE == WALK_FINAL ? *pass : 0.f;
    float P = 1.f;
    const float bias = by ? by[c] : 0.f;
    for (int j0 = 0; j0 < n; j0 += LRU_AHEAD) {
        float av[LRU_AHEAD], dv[LRU_AHEAD], yv[LRU_AHEAD];
#pragma unroll
        for (int k = 0; k < LRU_AHEAD; ++k) {  // a batch of loads, then the chain
            const int t = q0 + min(j0 + k, n - 1);
            av[k] = a[(size_t)t * C + c];
            dv[k] = drive[(size_t)t * C + c];
            if (MODE != WALK_LOCAL) yv[k] = to_f32(y[(size_t)t * ldy + ycol + c]);
        }
#pragma unroll
        for (int k = 0; k < LRU_AHEAD; ++k) {
            if (j0 + k < n) {
                S = av[k] * S + dv[k];
                if (MODE == WALK_LOCAL) P *= av[k];
                else out[(size_t)(q0 + j0 + k) * C + c] = from_f32<elem_t>(S * gelu_tanh_f(yv[k] + bias));
            }
        }
    }
    if (MODE == WALK_LOCAL) {
        pass[0] = P;
        pass[C] = S;
    } else if (last) {
        *st = S;
    }
}

// Between the two passes: S_in(seg + 1) = (product of seg's decays) * S_in(seg) + what seg adds, from the slot's state.
__global__ __launch_bounds__(256) void lru_carry_kernel(const float* __restrict__ state, const int* __restrict__ seq_q_len,
                                                        const int* __restrict__ seq_slot, float* __restrict__ carry, int C,
                                                        int seg_len, int n_segs) {
    const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int nseg = (seq_q_len[s] + seg_len - 1) / seg_len;
    float Sin = state[(size_t)seq_slot[s] * C + c];
    for (int seg = 0; seg < nseg; ++seg) {
        float* p = carry + ((size_t)s * n_segs + seg) * 2 * C + c;
        const bool more = seg + 1 < nseg;
        const float dec = more ? p[0] : 0.f, add = more ? p[C] : 0.f;
        p[0] = Sin;
        Sin = dec * Sin + add;
    }
}

// ---- the mix of a token with the one before it ---------------------------------------------
// out[m, t, :] = x[t] + (x[t - 1] - x[t]) * mu[m, :] for M mixes, in the element type; the row before a request's first
// row of the step comes from prev [slots, d] (zeros at the request's start).
__global__ __launch_bounds__(256) void shift_mix_kernel(const float* __restrict__ x, const float* __restrict__ prev,
                                                        const float* __restrict__ mu, int M, const int* __restrict__ seq_q_start,
                                                        const int* __restrict__ seq_slot, int S, elem_t* __restrict__ out, int T, int d) {
    const int t = blockIdx.x;
    const int s = seq_of_row(t, seq_q_start, S);
    const float* before = t > seq_q_start[s] ? x + (size_t)(t - 1) * d : prev + (size_t)seq_slot[s] * d;
    const float* cur = x + (size_t)t * d;
    const int c = blockIdx.y * 256 + threadIdx.x;
    if (c >= d) return;
    const float v = cur[c], dlt = before[c] - v;
    for (int m = 0; m < M; ++m) out[((size_t)m * T + t) * d + c] = from_f32<elem_t>(v + dlt * mu[(size_t)m * d + c]);
}

// prev[slot of request s] = its last row of the step
__global__ __launch_bounds__(256) void last_row_kernel(const float* __restrict__ x, float* __restrict__ prev,
                                                       const int* __restrict__ seq_q_start, const int* __restrict__ seq_q_len,
                                                       const int* __restrict__ seq_slot, int d) {
    const int s = blockIdx.x, n = seq_q_len[s];
    if (n <= 0) return;
    const float* src = x + (size_t)(seq_q_start[s] + n - 1) * d;
    float* dst = prev + (size_t)seq_slot[s] * d;
    for (int c = threadIdx.x; c < d; c += 256) dst[c] = src[c];
}

// out = act(in) in the element type: the bottleneck of a low-rank map between its two products (0: tanh)
__global__ __launch_bounds__(256) void tanh_rows_kernel(const float* __restrict__ in, elem_t* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = from_f32<elem_t>(tanhf(in[i]));
}

// ---- time mixing with a decay per key channel and token ----------------------------------------
// Per head, state S [d (key channel), d (value channel)]; token by token
//   o[j] = sum_i r[i] (S[i, j] + u[i] k[i] v[j]);   S[i, j] <- w[i] S[i, j] + k[i] v[j],   w = exp(-exp(z + w0)).
// A thread is a value channel j and holds its column of S in registers (DP of them, the head size rounded up to a
// multiple of 16; the rows beyond d stay zero).  The bonus is one number a token, sum_i r[i] u[i] k[i], times v[j].
// Then, in the same kernel: o / sqrt(mean_j o^2 + eps) * norm[h, j] * silu(gate[t, h, j]), rounded to the element type
// for the output projection.  Tokens come WKV_BATCH at a time: the next batch's numbers are asked for before the
// current batch is walked and put into LDS after it, so that the trip to memory runs beside the walk.
// A request's rows in one walk, or in segments side by side (see lru_scan_kernel): carry [S, n_segs, H, d, d] holds what
// a segment adds from zero and then the state that comes into it, cdec [S, n_segs, H, d] the product of its decays.
struct WkvArgs {
    const elem_t* r;     // [T, H * d]
    const elem_t* k;
    const elem_t* v;
    const elem_t* gate;  // [T, H * d] before its SiLU
    const float* z;      // [T, H * d]: the decay's inner logarithm before its offset
    const float* w0;     // [H * d]
    const float* u;      // [H * d]
    const float* norm;   // [H * d]
    float eps;
    float* state;        // [slots, H, d, d]
    const int* seq_q_start;
    const int* seq_q_len;
    const int* seq_slot;
    elem_t* out;         // [T, H * d]
    int H, d;
    int seg_len, n_segs;
    float* carry;
    float* cdec;
};

constexpr int WKV_BATCH = 8;

template <int DP, int MODE>
__global__ __launch_bounds__(DP <= 64 ? 64 : 128) void wkv_kernel(WkvArgs a) {
    constexpr int NT = DP <= 64 ? 64 : 128, NW = NT / 64, TB = WKV_BATCH;
    __shared__ __align__(16) float rs[TB][DP], ks[TB][DP], ws[TB][DP];
    __shared__ float vs[TB][NT], gs[TB][NT], bonus[TB][NW];
    __shared__ float os[TB][NT], halves[TB][2];
    const int s = blockIdx.x, h = blockIdx.y, seg = blockIdx.z, j = threadIdx.x, d = a.d, row = a.H * d;
    const int off = MODE == WALK_WHOLE ? 0 : seg * a.seg_len;
    const int left = a.seq_q_len[s] - off;
    if (left <= 0) return;
    const int n = MODE == WALK_WHOLE ? left : min(left, a.seg_len);
    const bool last = MODE == WALK_WHOLE || left <= a.seg_len;
    if (MODE == WALK_LOCAL && last) return;  // nobody needs what the last segment passes on
    const int q0 = a.seq_q_start[s] + off;
    const bool live = j < d;
    float* st = a.state + (((size_t)a.seq_slot[s] * a.H + h) * d) * d;
    float* pass = MODE == WALK_WHOLE ? nullptr : a.carry + ((((size_t)s * a.n_segs + seg) * a.H + h) * d) * d;
    float S[DP];
    {
        const float* from = MODE == WALK_FINAL ? pass : st;
#pragma unroll
        for (int i = 0; i < DP; ++i) S[i] = (MODE != WALK_LOCAL && live && i < d) ? from[(size_t)i * d + j] : 0.f;
    }
    const int col = h * d + (live ? j : 0);
    const float w0 = a.w0[col], uj = a.u[col], nw = a.norm[col];
    float pr[TB], pk[TB], pz[TB], pv[TB], pg[TB];
    auto fetch = [&](int j0) {  // this thread's channel of tokens j0 .. j0 + TB - 1 (the last one again beyond the end)
#pragma unroll
        for (int b = 0; b < TB; ++b) {
            const size_t at = (size_t)(q0 + min(j0 + b, n - 1)) * row + col;
            pk[b] = to_f32(a.k[at]);
            pz[b] = a.z[at];
            pv[b] = to_f32(a.v[at]);
            if (MODE != WALK_LOCAL) {
                pr[b] = to_f32(a.r[at]);
                pg[b] = to_f32(a.gate[at]);
            }
        }
    };
    float pw = 1.f;  // the product of this key channel's decays over the segment
    fetch(0);
    for (int j0 = 0; j0 < n; j0 += TB) {
        const int nb = min(TB, n - j0);
        __syncthreads();  // the batch before has been walked by everyone
#pragma unroll
        for (int b = 0; b < TB; ++b) {
            const float w = live ? expf(-expf(pz[b] + w0)) : 0.f;
            if (j < DP) {
                ks[b][j] = live ? pk[b] : 0.f;
                ws[b][j] = w;
            }
            vs[b][j] = live ? pv[b] : 0.f;
            if (MODE == WALK_LOCAL) {
                if (b < nb) pw *= w;
            } else {
                if (j < DP) rs[b][j] = live ? pr[b] : 0.f;
                gs[b][j] = pg[b];
                const float p = wave_sum(live ? pr[b] * uj * pk[b] : 0.f);
                if ((j & 63) == 0) bonus[b][j >> 6] = p;
            }
        }
        __syncthreads();
        if (j0 + TB < n) fetch(j0 + TB);
        // the batch's outputs wait in LDS, each in its thread's own place: their norms are worked out together behind the walk
#pragma unroll 1
        for (int b = 0; b < nb; ++b) {
            {
                const float vj = vs[b][j];
                float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;  // four chains of sums side by side
#pragma unroll
                for (int i = 0; i < DP; i += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(&ks[b][i]);
                    const float4 w4 = *reinterpret_cast<const float4*>(&ws[b][i]);
                    if (MODE != WALK_LOCAL) {
                        const float4 r4 = *reinterpret_cast<const float4*>(&rs[b][i]);
                        o0 = fmaf(r4.x, S[i], o0);
                        o1 = fmaf(r4.y, S[i + 1], o1);
                        o2 = fmaf(r4.z, S[i + 2], o2);
                        o3 = fmaf(r4.w, S[i + 3], o3);
                    }
                    S[i] = fmaf(w4.x, S[i], k4.x * vj);
                    S[i + 1] = fmaf(w4.y, S[i + 1], k4.y * vj);
                    S[i + 2] = fmaf(w4.z, S[i + 2], k4.z * vj);
                    S[i + 3] = fmaf(w4.w, S[i + 3], k4.w * vj);
                }
                if (MODE != WALK_LOCAL) {
                    float bn = bonus[b][0];
                    if constexpr (NW == 2) bn += bonus[b][1];
                    os[b][j] = fmaf(bn, vj, (o0 + o1) + (o2 + o3));
                }
            }
        }
        if (MODE != WALK_LOCAL) {
            float ob[TB], ss[TB];
#pragma unroll
            for (int b = 0; b < TB; ++b) {
                ob[b] = (live && b < nb) ? os[b][j] : 0.f;
                ss[b] = wave_sum(ob[b] * ob[b]);
            }
            if constexpr (NW == 2) {  // the head's other half
                __syncthreads();
                if ((j & 63) == 0) {
#pragma unroll
                    for (int b = 0; b < TB; ++b) halves[b][j >> 6] = ss[b];
                }
                __syncthreads();
#pragma unroll
                for (int b = 0; b < TB; ++b) ss[b] = halves[b][0] + halves[b][1];
            }
#pragma unroll
            for (int b = 0; b < TB; ++b) {
                if (live && b < nb) {
                    const float g = gs[b][j];
                    const float y = ob[b] / sqrtf(ss[b] / (float)d + a.eps) * nw * (g / (1.0f + expf(-g)));
                    a.out[(size_t)(q0 + j0 + b) * row + col] = from_f32<elem_t>(y);
                }
            }
        }
    }
    if (!live) return;
    if (MODE == WALK_LOCAL) {
#pragma unroll
        for (int i = 0; i < DP; ++i)
            if (i < d) pass[(size_t)i * d + j] = S[i];
        a.cdec[(((size_t)s * a.n_segs + seg) * a.H + h) * d + j] = pw;
    } else if (last) {
#pragma unroll
        for (int i = 0; i < DP; ++i)
            if (i < d) st[(size_t)i * d + j] = S[i];
    }
}

// Between the two passes: S_in(seg + 1) = diag(product of seg's decays) S_in(seg) + what seg adds, from the slot's state.
__global__ __launch_bounds__(256) void wkv_carry_kernel(const float* __restrict__ state, const int* __restrict__ seq_q_len,
                                                        const int* __restrict__ seq_slot, float* __restrict__ carry,
                                                        const float* __restrict__ cdec, int H, int d, int seg_len, int n_segs) {
    const int s = blockIdx.x, h = blockIdx.y, idx = blockIdx.z * 256 + threadIdx.x;
    if (idx >= d * d) return;
    const int i = idx / d;
    const int nseg = (seq_q_len[s] + seg_len - 1) / seg_len;
    float Sin = state[((size_t)seq_slot[s] * H + h) * d * d + idx];
    for (int seg = 0; seg < nseg; ++seg) {
        const size_t at = ((size_t)s * n_segs + seg) * H + h;
        float* p = carry + at * d * d + idx;
        const bool more = seg + 1 < nseg;
        const float dec = more ? cdec[at * d + i] : 0.f, add = more ? *p : 0.f;
        *p = Sin;
        Sin = dec * Sin + add;
    }
}

}  // namespace ms

using namespace ms;

extern "C" int ms_linrec_max_taps() { return MAX_TAPS; }
extern "C" int ms_wkv_max_dim() { return 128; }
extern "C" int ms_lru_max_block() { return 64 * 1024 / (GATE_ROWS * (int)sizeof(float)); }  // a block's rows lie in LDS

// One launch for the convolution and one for the state, in this order: the first reads the state that the second
// replaces.  `out` may not alias `in`.
extern "C" int ms_conv_sums(const float* in, int n_partials, long partial_stride, int ld, int col0, const float* bias_in, const float* w,
                            const float* bias_out, float* state, const int* seq_q_start, const int* seq_q_len, const int* seq_slot,
                            int S, float* out, int ld_out, int out0, int T, int C, int taps, hipStream_t stream) {
    MS_REQUIRE(T > 0 && C > 0 && S > 0 && n_partials > 0, "conv_sums: empty problem T=%d C=%d S=%d", T, C, S);
    MS_REQUIRE(taps >= 1 && taps <= MAX_TAPS, "conv_sums: %d taps (1 to %d)", taps, MAX_TAPS);
    MS_REQUIRE(col0 >= 0 && col0 + C <= ld && out0 >= 0 && out0 + C <= ld_out, "conv_sums: columns %d..%d of %d, %d..%d of %d", col0,
               col0 + C, ld, out0, out0 + C, ld_out);
    MS_REQUIRE(taps == 1 || state, "conv_sums: %d taps need a state", taps);
    ConvArgs a{in, n_partials, (size_t)partial_stride, ld, col0, bias_in, w, bias_out, state, seq_q_start, seq_q_len, seq_slot, S,
               out, ld_out, out0, C, taps};
    hipLaunchKernelGGL(conv_rows_kernel, dim3(T, ceil_div(C, 256)), dim3(256), 0, stream, a);
    int rc = check_launch("conv_sums");
    if (rc || taps == 1) return rc;
    hipLaunchKernelGGL(conv_rows_state_kernel, dim3(S, ceil_div(C, 256)), dim3(256), 0, stream, a);
    return check_launch("conv_sums_state");
}

extern "C" int ms_lru_gates(const float* u, const void* wa_t, const void* wi_t, const float* ba, const float* bi, const float* lam,
                            float c, float* a_out, float* drive_out, int T, int C, int blocks, hipStream_t stream) {
    MS_REQUIRE(T > 0 && C > 0 && blocks > 0 && C % blocks == 0, "lru_gates: %d channels in %d blocks, %d rows", C, blocks, T);
    const int bw = C / blocks;
    const size_t lds = (size_t)GATE_ROWS * ((bw + 3) & ~3) * sizeof(float);
    MS_REQUIRE(lds <= 64 * 1024, "lru_gates: blocks of %d channels exceed the rows' place in LDS", bw);
    GateArgs g{u, (const elem_t*)wa_t, (const elem_t*)wi_t, ba, bi, lam, c, a_out, drive_out, T, C, bw};
    hipLaunchKernelGGL(lru_gates_kernel, dim3(ceil_div(T, GATE_ROWS), blocks, ceil_div(bw, GATE_OUTS)), dim3(256), lds, stream, g);
    return check_launch("lru_gates");
}

// seg_len > 0: requests' rows in segments of seg_len that are walked side by side; n_segs covers the longest request of the
// step, carry holds [S, n_segs, 2, C] floats.
extern "C" int ms_lru_scan(const float* a, const float* drive, const void* y, int ldy, int ycol, const float* by, float* state,
                           const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, void* out, int C, int seg_len,
                           int n_segs, float* carry, hipStream_t stream) {
    MS_REQUIRE(S > 0 && C > 0 && ycol >= 0 && ycol + C <= ldy, "lru_scan: %d requests, %d channels at column %d of %d", S, C, ycol, ldy);
    MS_REQUIRE(seg_len == 0 || (seg_len > 0 && n_segs > 0 && carry), "lru_scan: segments of %d need their workspace", seg_len);
#define MS_LRU(MODE, Z)                                                                                                          \
    hipLaunchKernelGGL(lru_scan_kernel<MODE>, dim3(S, ceil_div(C, 64), Z), dim3(64), 0, stream, a, drive, (const elem_t*)y, ldy, \
                       ycol, by, state, seq_q_start, seq_q_len, seq_slot, (elem_t*)out, C, seg_len, n_segs, carry)
    if (seg_len == 0) {
        MS_LRU(WALK_WHOLE, 1);
        return check_launch("lru_scan");
    }
    MS_LRU(WALK_LOCAL, n_segs);
    if (int rc = check_launch("lru_scan, segments from zero")) return rc;
    hipLaunchKernelGGL(lru_carry_kernel, dim3(S, ceil_div(C, 256)), dim3(256), 0, stream, (const float*)state, seq_q_len, seq_slot,
                       carry, C, seg_len, n_segs);
    if (int rc = check_launch("lru_scan, states between segments")) return rc;
    MS_LRU(WALK_FINAL, n_segs);
#undef MS_LRU
    return check_launch("lru_scan, segments");
}

extern "C" int ms_shift_mix(const float* x, float* prev, const float* mu, int M, const int* seq_q_start, const int* seq_q_len,
                            const int* seq_slot, int S, void* out, int T, int d, hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0 && S > 0 && M > 0, "shift_mix: empty problem T=%d d=%d S=%d M=%d", T, d, S, M);
    hipLaunchKernelGGL(shift_mix_kernel, dim3(T, ceil_div(d, 256)), dim3(256), 0, stream, x, (const float*)prev, mu, M, seq_q_start, seq_slot, S,
                       (elem_t*)out, T, d);
    int rc = check_launch("shift_mix");
    if (rc) return rc;
    hipLaunchKernelGGL(last_row_kernel, dim3(S), dim3(256), 0, stream, x, prev, seq_q_start, seq_q_len, seq_slot, d);
    return check_launch("last_row");
}

extern "C" int ms_tanh_rows(const float* in, void* out, long n, hipStream_t stream) {
    MS_REQUIRE(n > 0, "tanh_rows: empty problem");
    hipLaunchKernelGGL(tanh_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, stream, in, (elem_t*)out, (size_t)n);
    return check_launch("tanh_rows");
}

// seg_len > 0: as for ms_lru_scan; carry holds [S, n_segs, H, d, d] floats and cdec [S, n_segs, H, d].
extern "C" int ms_wkv(const void* r, const void* k, const void* v, const void* gate, const float* z, const float* w0, const float* u,
                      const float* norm, float eps, float* state, const int* seq_q_start, const int* seq_q_len, const int* seq_slot,
                      int S, void* out, int H, int d, int seg_len, int n_segs, float* carry, float* cdec, hipStream_t stream) {
    MS_REQUIRE(S > 0 && H > 0 && d > 0 && d <= 128, "wkv: %d requests, %d heads of %d (at most 128)", S, H, d);
    MS_REQUIRE(seg_len == 0 || (seg_len > 0 && n_segs > 0 && carry && cdec), "wkv: segments of %d need their workspace", seg_len);
    WkvArgs a{(const elem_t*)r, (const elem_t*)k, (const elem_t*)v, (const elem_t*)gate, z, w0, u, norm, eps, state,
              seq_q_start, seq_q_len, seq_slot, (elem_t*)out, H, d, seg_len, n_segs, carry, cdec};
    const int dp = ceil_div(d, 16) * 16;
    auto walk = [&](auto mode, int Z) {
        constexpr int MODE = decltype(mode)::value;
        const dim3 grid(S, H, Z);
        switch (dp) {
            case 16: hipLaunchKernelGGL((wkv_kernel<16, MODE>), grid, dim3(64), 0, stream, a); break;
            case 32: hipLaunchKernelGGL((wkv_kernel<32, MODE>), grid, dim3(64), 0, stream, a); break;
            case 48: hipLaunchKernelGGL((wkv_kernel<48, MODE>), grid, dim3(64), 0, stream, a); break;
            case 64: hipLaunchKernelGGL((wkv_kernel<64, MODE>), grid, dim3(64), 0, stream, a); break;
            case 80: hipLaunchKernelGGL((wkv_kernel<80, MODE>), grid, dim3(128), 0, stream, a); break;
            case 96: hipLaunchKernelGGL((wkv_kernel<96, MODE>), grid, dim3(128), 0, stream, a); break;
            case 112: hipLaunchKernelGGL((wkv_kernel<112, MODE>), grid, dim3(128), 0, stream, a); break;
            default: hipLaunchKernelGGL((wkv_kernel<128, MODE>), grid, dim3(128), 0, stream, a); break;
        }
    };
    if (seg_len == 0) {
        walk(std::integral_constant<int, WALK_WHOLE>{}, 1);
        return check_launch("wkv");
    }
    walk(std::integral_constant<int, WALK_LOCAL>{}, n_segs);
    if (int rc = check_launch("wkv, segments from zero")) return rc;
    hipLaunchKernelGGL(wkv_carry_kernel, dim3(S, H, ceil_div(d * d, 256)), dim3(256), 0, stream, (const float*)state, seq_q_len,
                       seq_slot, carry, (const float*)cdec, H, d, seg_len, n_segs);
    if (int rc = check_launch("wkv, states between segments")) return rc;
    walk(std::integral_constant<int, WALK_FINAL>{}, n_segs);
    return check_launch("wkv, segments");
}
