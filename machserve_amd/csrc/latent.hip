// Attention through a latent (keys and values of every head are projections of one small vector per token).
//
// The cache keeps, per token, the normed latent c [rank] and one rotated key part [rot] that all heads share, as ONE
// key/value head of width rank + rot (filled with zeros up to the attention tile's multiple of 16).  A head's key is
// [W_uk_h c | rotated part] and its value W_uv_h c, so with q_h = [q_plain | q_rot]
//     score_h(i, j) = (W_uk_h^T q_plain_h(i)) . c(j) + q_rot_h(i) . k_rot(j),
//     out_h(i)      = W_uv_h (sum_j p_h(i, j) c(j)):
// the queries are carried into the latent's space by a product per head, the framework's paged attention kernels run
// over the cache with every query head in the one key/value head's group (each key is read once for all heads), and
// a second product per head carries the result out again.  Nothing of a head's keys or values is ever materialised.
//
// Kernels: the row kernel that finishes the down projections (two RMS norms with weights, the rotation of the shared
// key part by neighbouring pairs (2i, 2i + 1), the write into the page); the kernel that splits the up-projected
// queries into their plain part (operand of the per-head product) and their rotated part (written behind the
// latent's columns of the attention's queries); and the per-head product on the matrix cores.
// Norms, angles, cosines and sines are 32-bit in every build.
#include "common.cuh"

namespace ms {

struct LatentRowArgs {
    const float* proj;      // [n_partials, T, stride] partial sums of: query latent [q_rank], then (if kv) latent [rank], key part [rot]
    int n_partials;
    size_t partial_stride;
    int stride;
    const float* q_norm;    // [q_rank]
    const float* c_norm;    // [rank] or null: the layer reads another layer's cache and writes none
    float eps;
    const int* positions;   // [T]
    const float* inv_freq;  // [rot / 2]
    float cs_factor;        // what cosines and sines are multiplied by
    const int* slot_map;    // [T] page * ps + offset
    elem_t* cq_out;         // [T, cq_ld], zeros behind q_rank
    int cq_ld;
    elem_t* kpool;          // [pages, 1, ps, hd]
    elem_t* vpool;          // [pages, 1, hd, ps]
    int q_rank, rank, rot, hd, ps;
    int halves;             // the key part's pairs are (i, i + rot / 2), not (2i, 2i + 1)
};

// One block a row.  Columns of the key beyond rank + rot and rows of the value beyond rank are never written: the
// pools start as zeros and stay so there.
__global__ __launch_bounds__(256) void latent_row_kernel(LatentRowArgs a) {
    __shared__ float scratch[4];
    extern __shared__ float row[];  // stride floats
    const int t = blockIdx.x;
    const bool kv = a.c_norm != nullptr;
    const int n = a.q_rank + (kv ? a.rank + a.rot : 0);
    float ssq = 0.f, ssc = 0.f;
    // four columns a thread at a time, so that the loads of several columns and partial sums are in flight together
    for (int c0 = threadIdx.x; c0 < n; c0 += 1024) {
        float v[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
        for (int p = 0; p < a.n_partials; ++p) {
            const float* src = a.proj + p * a.partial_stride + (size_t)t * a.stride;
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] += src[min(c0 + u * 256, n - 1)];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int c = c0 + u * 256;
            if (c >= n) break;
            row[c] = v[u];
            if (c < a.q_rank) ssq += v[u] * v[u];
            else if (c < a.q_rank + a.rank) ssc += v[u] * v[u];
        }
    }
    ssq = block_sum<256>(ssq, scratch);
    ssc = block_sum<256>(ssc, scratch);
    __syncthreads();
    if (a.q_rank > 0) {  // 0: the queries have no bottleneck and are not this kernel's business
        const float inv_q = 1.0f / sqrtf(ssq / (float)a.q_rank + a.eps);
        for (int c = threadIdx.x; c < a.cq_ld; c += 256)
            a.cq_out[(size_t)t * a.cq_ld + c] = from_f32<elem_t>(c < a.q_rank ? row[c] * inv_q * a.q_norm[c] : 0.f);
    }
    if (!kv) return;
    const int slot = a.slot_map[t];
    if (slot < 0) return;
    const int page = slot / a.ps, off = slot % a.ps;
    const float inv_c = 1.0f / sqrtf(ssc / (float)a.rank + a.eps);
    elem_t* krow = a.kpool + ((size_t)page * a.ps + off) * a.hd;
    elem_t* vcol = a.vpool + (size_t)page * a.hd * a.ps + off;
    for (int c = threadIdx.x; c < a.rank; c += 256) {
        const elem_t v = from_f32<elem_t>(row[a.q_rank + c] * inv_c * a.c_norm[c]);
        krow[c] = v;
        vcol[(size_t)c * a.ps] = v;
    }
    const float pos = (float)a.positions[t];
    const float* kr = row + a.q_rank + a.rank;
    for (int i = threadIdx.x; i < a.rot / 2; i += 256) {
        float sn, cs;
        sincosf(pos * a.inv_freq[i], &sn, &cs);
        sn *= a.cs_factor;
        cs *= a.cs_factor;
        const int iu = a.halves ? i : 2 * i, iv = a.halves ? i + a.rot / 2 : 2 * i + 1;
        const float u = kr[iu], v = kr[iv];
        krow[a.rank + iu] = from_f32<elem_t>(u * cs - v * sn);
        krow[a.rank + iv] = from_f32<elem_t>(v * cs + u * sn);
    }
}

// q [T, H, d + rot] (32-bit sums of the up projection) -> plain [T, H, dp] in the element type (dp >= d, zeros behind d)
// and the rotated part into att [T, H, hd] at columns rank .. rank + rot, zeros behind it up to hd.
__global__ __launch_bounds__(256) void latent_query_kernel(const float* __restrict__ q, const int* __restrict__ positions,
                                                           const float* __restrict__ inv_freq, float cs_factor,
                                                           elem_t* __restrict__ plain, elem_t* __restrict__ att, int H, int d, int dp,
                                                           int rot, int rank, int hd, int halves) {
    const int t = blockIdx.x;
    const float pos = (float)positions[t];
    const float* qr = q + (size_t)t * H * (d + rot);
    for (int c = threadIdx.x; c < H * dp; c += 256) {
        const int h = c / dp, e = c - h * dp;
        plain[(size_t)t * H * dp + c] = from_f32<elem_t>(e < d ? qr[h * (d + rot) + e] : 0.f);
    }
    const int tail = hd - rank, half = rot / 2;  // per head: rot / 2 pairs, then single zeros
    const int units = half + (tail - rot);
    for (int c = threadIdx.x; c < H * units; c += 256) {
        const int h = c / units, i = c - h * units;
        elem_t* dst = att + ((size_t)t * H + h) * hd + rank;
        if (i < half) {
            float sn, cs;
            sincosf(pos * inv_freq[i], &sn, &cs);
            sn *= cs_factor;
            cs *= cs_factor;
            const int iu = halves ? i : 2 * i, iv = halves ? i + half : 2 * i + 1;
            const float u = qr[h * (d + rot) + d + iu], v = qr[h * (d + rot) + d + iv];
            dst[iu] = from_f32<elem_t>(u * cs - v * sn);
            dst[iv] = from_f32<elem_t>(v * cs + u * sn);
        } else {
            dst[rot + (i - half)] = from_f32<elem_t>(0.f);
        }
    }
}

// A product per head: out[t, b, n] = sum_k a[t, b, k] * w[b, n, k], with the rows of `a` and `out` strided (a head's
// part of a wider row), so that the result lands where its reader wants it.  Operands come straight from memory as
// fragments (a weight of one head is small and stays in the caches).  K is a multiple of 8; what lies beyond it, or
// beyond the last row or column, is read as zero.
struct HeadsLinearArgs {
    const elem_t* a;
    const elem_t* w;  // [B, N, K]
    elem_t* out;
    int T, B, N, K;
    long lda, a_head;  // element strides of a row and of a head in `a`
    long ldo, o_head;  // the same in `out`
};

// RT row tiles and CT column tiles of 16 a wave.  WAVES_OVER_ROWS: the block's four waves lie along the rows (a block is
// 64 * RT rows by 16 * CT columns), else along the columns (16 * RT rows by 64 * CT columns).
template <int RT, int CT, bool WAVES_OVER_ROWS>
__global__ __launch_bounds__(256) void heads_linear_kernel(HeadsLinearArgs g) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int r16 = lane & 15, grp = lane >> 4;
    const int b = blockIdx.z;
    const int row0 = (WAVES_OVER_ROWS ? blockIdx.x * 4 + wave : blockIdx.x) * 16 * RT;
    const int col0 = (WAVES_OVER_ROWS ? blockIdx.y : blockIdx.y * 4 + wave) * 16 * CT;
    if (row0 >= g.T || col0 >= g.N) return;  // the same for the whole wave; there is no barrier below
    const elem_t* ab = g.a + (size_t)b * g.a_head;
    const elem_t* wb = g.w + (size_t)b * g.N * g.K;
    f32x4 acc[RT][CT];
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    for (int k0 = 0; k0 < g.K; k0 += 32) {
        const int k = k0 + grp * 8;
        const bool k_in = k < g.K;
        Frag af[RT], bf[CT];
#pragma unroll
        for (int i = 0; i < RT; ++i) {
            const int row = row0 + i * 16 + r16;
            af[i] = (k_in && row < g.T) ? frag_load(ab + (size_t)row * g.lda + k) : frag_zero();
        }
#pragma unroll
        for (int j = 0; j < CT; ++j) {
            const int col = col0 + j * 16 + r16;
            bf[j] = (k_in && col < g.N) ? frag_load(wb + (size_t)col * g.K + k) : frag_zero();
        }
#pragma unroll
        for (int i = 0; i < RT; ++i)
#pragma unroll
            for (int j = 0; j < CT; ++j) mma_16x16x32(acc[i][j], af[i], bf[j]);
    }
#pragma unroll
    for (int i = 0; i < RT; ++i)
#pragma unroll
        for (int j = 0; j < CT; ++j) {
            const int col = col0 + j * 16 + r16;
            if (col >= g.N) continue;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int r = row0 + i * 16 + grp * 4 + e;
                if (r < g.T) g.out[(size_t)r * g.ldo + (size_t)b * g.o_head + col] = from_f32<elem_t>(acc[i][j][e]);
            }
        }
}

// out[i] = sigmoid(in[i]): a gate per row and head from 32-bit sums
__global__ __launch_bounds__(256) void sigmoid_rows_kernel(const float* __restrict__ in, float* __restrict__ out, long n) {
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) out[i] = 1.0f / (1.0f + expf(-in[i]));
}

}  // namespace ms

using namespace ms;

constexpr int LATENT_MAX_ROW = 15000;  // floats of a row of the down projections that a block holds in LDS
extern "C" int ms_latent_max_row() { return LATENT_MAX_ROW; }

// proj: float [n_partials, T, stride].  c_norm null: only the query latent is finished (the layer reads another
// layer's cache); then slot_map, kpool, vpool, inv_freq are not read.
extern "C" int ms_latent_rows(const float* proj, int n_partials, int stride, const float* q_norm, const float* c_norm, float eps,
                              const int* positions, const float* inv_freq, float cs_factor, const int* slot_map, void* cq_out,
                              int cq_ld, void* kpool, void* vpool, int T, int q_rank, int rank, int rot, int hd, int ps, int halves,
                              hipStream_t stream) {
    MS_REQUIRE(T > 0 && n_partials >= 1 && q_rank >= 0 && cq_ld >= q_rank, "latent rows: %d rows, %d partial sums, query latent of %d in %d", T, n_partials, q_rank, cq_ld);
    MS_REQUIRE(q_rank > 0 || c_norm, "latent rows: neither a query latent nor a cache to write");
    const int n = q_rank + (c_norm ? rank + rot : 0);
    MS_REQUIRE(stride >= n && n <= LATENT_MAX_ROW, "latent rows: a row of %d numbers (stride %d, at most %d)", n, stride, LATENT_MAX_ROW);
    if (c_norm) {
        MS_REQUIRE(rank > 0 && rot >= 0 && rot % 2 == 0 && rank + rot <= hd, "latent rows: latent %d + rotated part %d in a key of %d", rank, rot, hd);
        MS_REQUIRE(positions && slot_map && kpool && vpool && (rot == 0 || inv_freq), "latent rows: the layer writes the cache");
    }
    LatentRowArgs a{proj, n_partials, (size_t)T * stride, stride, q_norm, c_norm, eps, positions, inv_freq, cs_factor, slot_map,
                    (elem_t*)cq_out, cq_ld, (elem_t*)kpool, (elem_t*)vpool, q_rank, rank, rot, hd, ps, halves};
    hipLaunchKernelGGL(latent_row_kernel, dim3(T), dim3(256), (size_t)n * sizeof(float), stream, a);
    return check_launch("latent_rows");
}

extern "C" int ms_latent_query(const float* q, const int* positions, const float* inv_freq, float cs_factor, void* plain, void* att,
                               int T, int H, int d, int dp, int rot, int rank, int hd, int halves, hipStream_t stream) {
    MS_REQUIRE(T > 0 && H > 0 && d > 0 && dp >= d, "latent query: %d rows, %d heads, plain part %d in %d", T, H, d, dp);
    MS_REQUIRE(rot >= 0 && rot % 2 == 0 && rank + rot <= hd && (rot == 0 || inv_freq), "latent query: latent %d + rotated part %d in a key of %d", rank, rot, hd);
    hipLaunchKernelGGL(latent_query_kernel, dim3(T), dim3(256), 0, stream, q, positions, inv_freq, cs_factor, (elem_t*)plain,
                       (elem_t*)att, H, d, dp, rot, rank, hd, halves);
    return check_launch("latent_query");
}

extern "C" int ms_heads_linear(const void* a, long lda, long a_head, const void* w, void* out, long ldo, long o_head, int T, int B, int N,
                               int K, hipStream_t stream) {
    MS_REQUIRE(T > 0 && B > 0 && N > 0 && K > 0, "heads_linear: empty problem T=%d B=%d N=%d K=%d", T, B, N, K);
    MS_REQUIRE(K % 8 == 0 && lda % 8 == 0 && a_head % 8 == 0, "heads_linear: K = %d and the strides of the input (%ld, %ld) must be multiples of 8", K, lda, a_head);
    MS_REQUIRE(B <= 65535, "heads_linear: %d heads", B);
    MS_REQUIRE((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(w)) % 16 == 0, "heads_linear: operands must be 16-byte aligned");
    HeadsLinearArgs g{(const elem_t*)a, (const elem_t*)w, (elem_t*)out, T, B, N, K, lda, a_head, ldo, o_head};
    if (T >= 256) {  // a wave 64 rows by 64 columns: a weight fragment feeds four products
        hipLaunchKernelGGL((heads_linear_kernel<4, 4, true>), dim3(ceil_div(T, 256), ceil_div(N, 64), B), dim3(256), 0, stream, g);
    } else if (T > 16) {
        hipLaunchKernelGGL((heads_linear_kernel<1, 4, true>), dim3(ceil_div(T, 64), ceil_div(N, 64), B), dim3(256), 0, stream, g);
    } else {        // few rows: a wave one tile of 16 columns, so that the heads' weights are spread over many waves
        hipLaunchKernelGGL((heads_linear_kernel<1, 1, false>), dim3(1, ceil_div(N, 64), B), dim3(256), 0, stream, g);
    }
    return check_launch("heads_linear");
}

extern "C" int ms_sigmoid_rows(const float* in, float* out, long n, hipStream_t stream) {
    MS_REQUIRE(n > 0 && in && out, "sigmoid_rows: %ld numbers", n);
    hipLaunchKernelGGL(sigmoid_rows_kernel, dim3((unsigned)std::min<long>(ceil_div(n, 256L), 4096L)), dim3(256), 0, stream, in, out, n);
    return check_launch("sigmoid_rows");
}
