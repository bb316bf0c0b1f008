// The second Mamba layer's recurrence (state-space duality) and the gated norm behind it.
//
// Per request, head h and token t, with x [P] the head's value channels, B and C [N] those of the head's group, all
// behind a convolution (32-bit rows) and SiLU, which is applied here where they are read:
//     dt = softplus(raw_dt[t, h] + dt_bias[h]);   a = exp(-exp(A_log[h]) dt)
//     S <- a S + dt B x^T   (S is N x P, 32-bit, carried in the request's slot);   y = S^T C + D[h] x
// A block walks one (request, head): a thread owns one value channel and keeps its column of the state in registers;
// the tokens' B, C, step sizes and decays come through LDS a few tokens at a time, so every thread reads them as
// broadcasts.  Everything is 32-bit in every build.
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
};

template <int NMAX>
__global__ __launch_bounds__(256) void ssd_scan_kernel(SsdArgs a) {
    extern __shared__ float lds[];  // B [TOK, N], C [TOK, N], dt [TOK], decay [TOK]
    float* Bs = lds;
    float* Cs = lds + SSD_TOK * a.N;
    float* dts = Cs + SSD_TOK * a.N;
    float* decs = dts + SSD_TOK;
    const int s = blockIdx.x, h = blockIdx.y, p = threadIdx.x;
    const int n_rows = a.seq_q_len[s];
    if (n_rows <= 0) return;  // the same for the whole block
    const int row0 = a.seq_q_start[s], slot = a.seq_slot[s];
    const int g = h / (a.H / a.G);
    const bool live = p < a.P;
    const int inner = a.H * a.P;
    float* st = a.state + ((size_t)slot * a.H + h) * a.N * a.P + p;
    float S[NMAX];
#pragma unroll
    for (int n = 0; n < NMAX; ++n) S[n] = (live && n < a.N) ? st[(size_t)n * a.P] : 0.f;
    const float rate = expf(a.a_log[h]), bias = a.dt_bias[h], skip = a.d_skip[h];
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
            Bs[i] = silu_f(src[0]);
            Cs[i] = silu_f(src[(size_t)a.G * a.N]);
        }
        if (threadIdx.x < nt) {
            const float dt = softplus_f(a.proj[(size_t)(row0 + t0 + threadIdx.x) * a.ld_proj + a.dt_col + h] + bias);
            dts[threadIdx.x] = dt;
            decs[threadIdx.x] = expf(-rate * dt);
        }
        __syncthreads();
        for (int k = 0; k < nt; ++k) {
            const float dec = decs[k], dx = dts[k] * xv[k];
            const float* Bk = Bs + k * a.N;
            const float* Ck = Cs + k * a.N;
            float acc0 = 0.f, acc1 = 0.f;
#pragma unroll
            for (int n = 0; n < NMAX; n += 2) {
                if (n < a.N) {
                    S[n] = dec * S[n] + dx * Bk[n];
                    acc0 += S[n] * Ck[n];
                }
                if (n + 1 < a.N) {
                    S[n + 1] = dec * S[n + 1] + dx * Bk[n + 1];
                    acc1 += S[n + 1] * Ck[n + 1];
                }
            }
            if (live) a.y[(size_t)(row0 + t0 + k) * inner + h * a.P + p] = acc0 + acc1 + skip * xv[k];
        }
    }
    if (live) {
#pragma unroll
        for (int n = 0; n < NMAX; ++n)
            if (n < a.N) st[(size_t)n * a.P] = S[n];
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

extern "C" int ms_ssd_scan(const float* xbc, int ld_xbc, const float* proj, int ld_proj, int dt_col, const float* dt_bias, const float* a_log,
                           const float* d_skip, float* state, const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, float* y,
                           int T, int H, int P, int N, int G, hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && H > 0 && G > 0 && H % G == 0, "ssd_scan: %d rows of %d requests, %d heads in %d groups", T, S, H, G);
    MS_REQUIRE(P >= 1 && P <= SSD_MAX_HEAD && N >= 1 && N <= SSD_MAX_STATES, "ssd_scan: heads of %d (at most %d) with %d states (at most %d)", P,
               SSD_MAX_HEAD, N, SSD_MAX_STATES);
    MS_REQUIRE(ld_xbc >= H * P + 2 * G * N && ld_proj >= dt_col + H && dt_col >= 0, "ssd_scan: rows of %d and %d numbers for %d heads", ld_xbc,
               ld_proj, H);
    SsdArgs a{xbc, ld_xbc, proj, ld_proj, dt_col, dt_bias, a_log, d_skip, state, seq_q_start, seq_q_len, seq_slot, y, H, P, N, G};
    const dim3 grid(S, H), block(ceil_div(P, 64) * 64);
    const size_t lds = (size_t)(2 * SSD_TOK * N + 2 * SSD_TOK) * sizeof(float);
    if (N <= 16) hipLaunchKernelGGL(ssd_scan_kernel<16>, grid, block, lds, stream, a);
    else if (N <= 32) hipLaunchKernelGGL(ssd_scan_kernel<32>, grid, block, lds, stream, a);
    else if (N <= 64) hipLaunchKernelGGL(ssd_scan_kernel<64>, grid, block, lds, stream, a);
    else if (N <= 128) hipLaunchKernelGGL(ssd_scan_kernel<128>, grid, block, lds, stream, a);
    else hipLaunchKernelGGL(ssd_scan_kernel<256>, grid, block, lds, stream, a);
    return check_launch("ssd_scan");
}

extern "C" int ms_gated_group_norm(const float* y, const float* z, int ld_z, const float* w, void* out, int ld_out, int T, int n, int parts,
                                   float eps, hipStream_t stream) {
    MS_REQUIRE(T > 0 && n > 0 && parts >= 1 && n % parts == 0 && ld_out >= n && ld_z >= n, "gated_group_norm: %d rows of %d in %d parts", T, n, parts);
    MS_REQUIRE(parts <= 65535, "gated_group_norm: %d parts", parts);
    hipLaunchKernelGGL(gated_group_norm_kernel, dim3(T, parts), dim3(256), 0, stream, y, z, ld_z, w, (elem_t*)out, ld_out, n, parts, eps);
    return check_launch("gated_group_norm");
}
