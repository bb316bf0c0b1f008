// The second Mamba layer's recurrence (state-space duality) and the gated norm behind it.
//
// Per request, head h and token t, with x [P] the head's value channels, B and C [N] those of the head's group, all
// behind a convolution (32-bit rows) and SiLU, which is applied here where they are read:
//     dt = softplus(raw_dt[t, h] + dt_bias[h]);   a = exp(-exp(A_log[h]) dt)
//     S <- a S + dt B x^T   (S is N x P, 32-bit, carried in the request's slot);   y = S^T C + D[h] x
// A block walks one (request, head): a thread owns one value channel and keeps its column of the state in registers;
// the tokens' B, C, step sizes and decays come through LDS a few tokens at a time, so every thread reads them as
// broadcasts, four states at once.  Long portions are cut into segments that are walked side by side (see the kernel).
// Everything is 32-bit in every build.
#include "common.cuh"

namespace ms {

constexpr int SSD_TOK = 8;  // tokens whose B, C, dt and decay a block holds in LDS at a time

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

struct SsdArgs {
    const float* xbc;      // [T, ld_xbc]: x [H, P], B [G, N], C [G, N] before their SiLU
    int ld_xbc;
    const float* proj;     // [T, ld_proj]: column dt_col + h is head h's raw step size
    int ld_proj, dt_col;
    const float* dt_bias;  // [H]
    const float* a_log;    // [H]
    const float* d_skip;   // [H]
    float* state;          // [slots, H, N, P]
    const int* seq_q_start;
    const int* seq_q_len;
    const int* seq_slot;
    float* y;              // [T, H * P]
    int H, P, N, G;
    int seg_len, n_segs;   // a request's rows in segments walked side by side (0: one walk)
    float* carry;          // [S, n_segs, H, N, P]: what a segment adds from zero, then the state that comes into it
    float* cdec;           // [S, n_segs, H]: the product of a segment's decays
};

// A request's rows in one walk (WHOLE), or in segments side by side: every segment but a request's last is first walked
// from zero (LOCAL: what it adds to the state and the product of its decays, no output), a carry kernel chains
// S_in(seg + 1) = D_seg S_in(seg) + add_seg from the slot's state, and every segment is walked again from its own S_in
// (FINAL), token after token.  Within a segment the order is the token order.
constexpr int SSD_WHOLE = 0, SSD_LOCAL = 1, SSD_FINAL = 2;

template <int NMAX, int MODE>
__global__ __launch_bounds__(256) void ssd_scan_kernel(SsdArgs a) {
    extern __shared__ __align__(16) float lds[];  // B [TOK, NMAX], C [TOK, NMAX] (zeros beyond N), dt [TOK], decay [TOK]
    float* Bs = lds;
    float* Cs = lds + SSD_TOK * NMAX;
    float* dts = Cs + SSD_TOK * NMAX;
    float* decs = dts + SSD_TOK;
    const int s = blockIdx.x, h = blockIdx.y, seg = blockIdx.z, p = threadIdx.x;
    const int off = MODE == SSD_WHOLE ? 0 : seg * a.seg_len;
    const int left = a.seq_q_len[s] - off;
    if (left <= 0) return;  // the same for the whole block
    const int n_rows = MODE == SSD_WHOLE ? left : min(left, a.seg_len);
    const bool last = MODE == SSD_WHOLE || left <= a.seg_len;
    if (MODE == SSD_LOCAL && last) return;  // nobody needs what the last segment passes on
    const int row0 = a.seq_q_start[s] + off, slot = a.seq_slot[s];
    const int g = h / (a.H / a.G);
    const bool live = p < a.P;
    const int inner = a.H * a.P;
    float* st = a.state + ((size_t)slot * a.H + h) * a.N * a.P + p;
    float* pass = MODE == SSD_WHOLE ? nullptr : a.carry + (((size_t)s * a.n_segs + seg) * a.H + h) * a.N * a.P + p;
    float S[NMAX];
    {
        const float* from = MODE == SSD_FINAL ? pass : st;
#pragma unroll
        for (int n = 0; n < NMAX; ++n) S[n] = (MODE != SSD_LOCAL && live && n < a.N) ? from[(size_t)n * a.P] : 0.f;
    }
    const float rate = expf(a.a_log[h]), bias = a.dt_bias[h], skip = a.d_skip[h];
    float prod = 1.f;
    for (int i = threadIdx.x; i < 2 * SSD_TOK * NMAX; i += blockDim.x) lds[i] = 0.f;  // the columns beyond N stay zeros
    for (int t0 = 0; t0 < n_rows; t0 += SSD_TOK) {
        const int nt = min(SSD_TOK, n_rows - t0);
        float xv[SSD_TOK];
#pragma unroll
        for (int k = 0; k < SSD_TOK; ++k)
            xv[k] = (live && k < nt) ? silu_f(a.xbc[(size_t)(row0 + t0 + k) * a.ld_xbc + h * a.P + p]) : 0.f;
        __syncthreads();  // the tile before has been read
        for (int i = threadIdx.x; i < nt * a.N; i += blockDim.x) {
            const int k = i / a.N, n = i - k * a.N;
            const float* src = a.xbc + (size_t)(row0 + t0 + k) * a.ld_xbc + inner + g * a.N + n;
            Bs[k * NMAX + n] = silu_f(src[0]);
            if (MODE != SSD_LOCAL) Cs[k * NMAX + n] = silu_f(src[(size_t)a.G * a.N]);
        }
        if (threadIdx.x < nt) {
            const float dt = softplus_f(a.proj[(size_t)(row0 + t0 + threadIdx.x) * a.ld_proj + a.dt_col + h] + bias);
            dts[threadIdx.x] = dt;
            decs[threadIdx.x] = expf(-rate * dt);
        }
        __syncthreads();
        for (int k = 0; k < nt; ++k) {
            const float dec = decs[k], dx = dts[k] * xv[k];
            const float4* Bk = reinterpret_cast<const float4*>(Bs + k * NMAX);
            const float4* Ck = reinterpret_cast<const float4*>(Cs + k * NMAX);
            float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
#pragma unroll
            for (int n = 0; n < NMAX; n += 4) {
                const float4 b = Bk[n >> 2];
                S[n] = dec * S[n] + dx * b.x;
                S[n + 1] = dec * S[n + 1] + dx * b.y;
                S[n + 2] = dec * S[n + 2] + dx * b.z;
                S[n + 3] = dec * S[n + 3] + dx * b.w;
                if (MODE != SSD_LOCAL) {
                    const float4 c = Ck[n >> 2];
                    acc0 += S[n] * c.x;
                    acc1 += S[n + 1] * c.y;
                    acc2 += S[n + 2] * c.z;
                    acc3 += S[n + 3] * c.w;
                }
            }
            if (MODE == SSD_LOCAL) prod *= dec;
            else if (live) a.y[(size_t)(row0 + t0 + k) * inner + h * a.P + p] = (acc0 + acc1) + (acc2 + acc3) + skip * xv[k];
        }
    }
    if (MODE == SSD_LOCAL) {
        if (live) {
#pragma unroll
            for (int n = 0; n < NMAX; ++n)
                if (n < a.N) pass[(size_t)n * a.P] = S[n];
        }
        if (threadIdx.x == 0) a.cdec[((size_t)s * a.n_segs + seg) * a.H + h] = prod;
    } else if (last && live) {
#pragma unroll
        for (int n = 0; n < NMAX; ++n)
            if (n < a.N) st[(size_t)n * a.P] = S[n];
    }
}

// Between the two passes: S_in(seg + 1) = (product of seg's decays) * S_in(seg) + what seg adds, from the slot's state.
__global__ __launch_bounds__(256) void ssd_carry_kernel(SsdArgs a) {
    const int s = blockIdx.x, h = blockIdx.y, i = blockIdx.z * 256 + threadIdx.x, np = a.N * a.P;
    if (i >= np) return;
    const int nseg = (a.seq_q_len[s] + a.seg_len - 1) / a.seg_len;
    float Sin = a.state[((size_t)a.seq_slot[s] * a.H + h) * np + i];
    for (int seg = 0; seg < nseg; ++seg) {
        float* p = a.carry + (((size_t)s * a.n_segs + seg) * a.H + h) * np + i;
        const bool more = seg + 1 < nseg;
        const float dec = more ? a.cdec[((size_t)s * a.n_segs + seg) * a.H + h] : 0.f, add = more ? *p : 0.f;
        *p = Sin;
        Sin = dec * Sin + add;
    }
}

// out[t, c] = (y[t, c] silu(z[t, c])) / sqrt(mean over c's part of the same squared + eps) * w[c], in the element type;
// the row has `parts` equal parts, each normed by itself; columns n .. ld_out of the output are zeros.
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const float* __restrict__ z, int ld_z,
                                                               const float* __restrict__ w, elem_t* __restrict__ out, int ld_out, int n,
                                                               int parts, float eps) {
    __shared__ float scratch[4];
    const int t = blockIdx.x, part = blockIdx.y, m = n / parts, c0 = part * m;
    const float* yr = y + (size_t)t * n + c0;
    const float* zr = z + (size_t)t * ld_z + c0;
    float ss = 0.f;
    for (int c = threadIdx.x; c < m; c += 256) {
        const float v = yr[c] * silu_f(zr[c]);
        ss += v * v;
    }
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)m + eps);
    for (int c = threadIdx.x; c < m; c += 256)
        out[(size_t)t * ld_out + c0 + c] = from_f32<elem_t>(yr[c] * silu_f(zr[c]) * inv * w[c0 + c]);
    if (part == 0)
        for (int c = n + threadIdx.x; c < ld_out; c += 256) out[(size_t)t * ld_out + c] = from_f32<elem_t>(0.f);
}

}  // namespace ms

using namespace ms;

constexpr int SSD_MAX_STATES = 256, SSD_MAX_HEAD = 256;
extern "C" int ms_ssd_max_states() { return SSD_MAX_STATES; }
extern "C" int ms_ssd_max_head() { return SSD_MAX_HEAD; }

template <int MODE>
static void launch_ssd(const SsdArgs& a, int S, int Z, hipStream_t stream) {
    const dim3 grid(S, a.H, Z), block(ceil_div(a.P, 64) * 64);
#define MS_SSD(NMAX) hipLaunchKernelGGL((ssd_scan_kernel<NMAX, MODE>), grid, block, (size_t)(2 * SSD_TOK * NMAX + 2 * SSD_TOK) * sizeof(float), stream, a)
    if (a.N <= 16) MS_SSD(16);
    else if (a.N <= 32) MS_SSD(32);
    else if (a.N <= 64) MS_SSD(64);
    else if (a.N <= 128) MS_SSD(128);
    else MS_SSD(256);
#undef MS_SSD
}

// seg_len 0: every request's rows in one walk.  Else carry float [S, n_segs, H, N, P] and cdec float [S, n_segs, H] are
// the workspace of the segments.
extern "C" int ms_ssd_scan(const float* xbc, int ld_xbc, const float* proj, int ld_proj, int dt_col, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, float* y,
                           int T, int H, int P, int N, int G, int seg_len, int n_segs, float* carry, float* cdec, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && H > 0 && G > 0 && H % G == 0, "ssd_scan: %d rows of %d requests, %d heads in %d groups", T, S, H, G);
    MS_REQUIRE(P >= 1 && P <= SSD_MAX_HEAD && N >= 1 && N <= SSD_MAX_STATES, "ssd_scan: heads of %d (at most %d) with %d states (at most %d)", P,
               SSD_MAX_HEAD, N, SSD_MAX_STATES);
    MS_REQUIRE(ld_xbc >= H * P + 2 * G * N && ld_proj >= dt_col + H && dt_col >= 0, "ssd_scan: rows of %d and %d numbers for %d heads", ld_xbc,
               ld_proj, H);
    MS_REQUIRE(H <= 65535 && n_segs <= 65535, "ssd_scan: %d heads, %d segments", H, n_segs);
    MS_REQUIRE(seg_len == 0 || (seg_len > 0 && n_segs > 1 && carry && cdec), "ssd_scan: segments of %d rows, %d a request, without their workspace", seg_len, n_segs);
    SsdArgs a{xbc, ld_xbc, proj, ld_proj, dt_col, dt_bias, a_log, d_skip, state, seq_q_start, seq_q_len, seq_slot, y, H, P, N, G, seg_len, n_segs, carry, cdec};
    if (seg_len == 0) {
        launch_ssd<SSD_WHOLE>(a, S, 1, stream);
        return check_launch("ssd_scan");
    }
    launch_ssd<SSD_LOCAL>(a, S, n_segs, stream);
    if (int rc = check_launch("ssd_scan, segments from zero")) return rc;
    hipLaunchKernelGGL(ssd_carry_kernel, dim3(S, H, ceil_div(N * P, 256)), dim3(256), 0, stream, a);
    if (int rc = check_launch("ssd_scan, states between segments")) return rc;
    launch_ssd<SSD_FINAL>(a, S, n_segs, stream);
    return check_launch("ssd_scan, segments");
}

extern "C" int ms_gated_group_norm(const float* y, const float* z, int ld_z, const float* w, void* out, int ld_out, int T, int n, int parts,
                                   float eps, hipStream_t stream) {
    MS_REQUIRE(T > 0 && n > 0 && parts >= 1 && n % parts == 0 && ld_out >= n && ld_z >= n, "gated_group_norm: %d rows of %d in %d parts", T, n, parts);
    MS_REQUIRE(parts <= 65535, "gated_group_norm: %d parts", parts);
    hipLaunchKernelGGL(gated_group_norm_kernel, dim3(T, parts), dim3(256), 0, stream, y, z, ld_z, w, (elem_t*)out, ld_out, n, parts, eps);
    return check_launch("gated_group_norm");
}
