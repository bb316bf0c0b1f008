// Several residual streams xs [streams, T, d] (32-bit): a branch reads a weighted sum of them and is written back into
// all of them at once.
//
//   read:   u[t] = sum_s w_in[s] xs[s, t]                       (w_in null: the plain sum; of chosen rows if asked)
//           with a norm: h[t] = u[t] / sqrt(mean(u[t]^2) + eps) * w, in the element type, the same kernel
//   write:  y[t] = sum_p sums[p, t] + bias;   xs[s', t] <- sum_s mix[s, s'] xs[s, t] + w_out[s'] y[t]   for all s' at once
//   write and read: a write and the next branch's read with its norm in one kernel (a block a row), which saves the read's
//           pass over the streams: the new values are summed with the next weights while they are in registers
//
// The write kernel adds up the partial sums that a branch's last product left, so that product needs no pass of its own
// over the streams.  Every thread reads the old values of its columns in all streams before it writes any of them.
#include "common.cuh"

namespace ms {

constexpr int MAX_STREAMS = 8;

struct StreamsReadArgs {
    const float* xs;       // [S, T, d]
    const float* w_in;     // [S] or null
    const int* rows;       // [R] rows to read, or null: all T
    const float* norm_w;   // [d] (NORM)
    float eps;
    float* out_f32;        // [R, d] (no norm)
    elem_t* out;           // [R, d] (NORM)
    int S, T, d;
};

template <bool NORM>
__global__ __launch_bounds__(256) void streams_read_kernel(StreamsReadArgs a) {
    __shared__ float scratch[4];
    extern __shared__ float row[];  // d floats (NORM)
    const int r = blockIdx.x;
    const int t = a.rows ? a.rows[r] : r;
    float w[MAX_STREAMS];
#pragma unroll
    for (int s = 0; s < MAX_STREAMS; ++s) w[s] = s < a.S ? (a.w_in ? a.w_in[s] : 1.0f) : 0.f;
    const size_t plane = (size_t)a.T * a.d;
    const float* src = a.xs + (size_t)t * a.d;
    float ss = 0.f;
    if ((a.d & 3) == 0) {
        for (int c = threadIdx.x * 4; c < a.d; c += 1024) {
            float4 u = (float4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s) {
                if (s >= a.S) break;
                const float4 v = *reinterpret_cast<const float4*>(src + s * plane + c);
                u.x += w[s] * v.x; u.y += w[s] * v.y; u.z += w[s] * v.z; u.w += w[s] * v.w;
            }
            if constexpr (NORM) {
                *reinterpret_cast<float4*>(row + c) = u;
                ss += u.x * u.x + u.y * u.y + u.z * u.z + u.w * u.w;
            } else {
                *reinterpret_cast<float4*>(a.out_f32 + (size_t)r * a.d + c) = u;
            }
        }
    } else {
        for (int c = threadIdx.x; c < a.d; c += 256) {
            float u = 0.f;
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s) {
                if (s >= a.S) break;
                u += w[s] * src[s * plane + c];
            }
            if constexpr (NORM) {
                row[c] = u;
                ss += u * u;
            } else {
                a.out_f32[(size_t)r * a.d + c] = u;
            }
        }
    }
    if constexpr (NORM) {
        ss = block_sum<256>(ss, scratch);
        const float inv = 1.0f / sqrtf(ss / (float)a.d + a.eps);
        for (int c = threadIdx.x; c < a.d; c += 256) a.out[(size_t)r * a.d + c] = from_f32<elem_t>(row[c] * inv * a.norm_w[c]);
    }
}

struct StreamsWriteArgs {
    float* xs;            // [S, T, d], rewritten in place
    const float* sums;    // [P, T, d]
    const float* bias;    // [d] or null
    const float* mix;     // [S, S], indexed [from, to]
    const float* w_out;   // [S]
    int P, S, T, d;
};

template <int V>  // columns a thread takes at once
__global__ __launch_bounds__(256) void streams_write_kernel(StreamsWriteArgs a) {
    __shared__ float m[MAX_STREAMS * MAX_STREAMS + MAX_STREAMS];
    for (int i = threadIdx.x; i < a.S * a.S + a.S; i += 256) m[i] = i < a.S * a.S ? a.mix[i] : a.w_out[i - a.S * a.S];
    __syncthreads();
    const size_t plane = (size_t)a.T * a.d;
    const long n = (long)plane / V;
    for (long i = (long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long)gridDim.x * 256) {
        const size_t at = (size_t)i * V;
        const int c = (int)(at % a.d);
        float y[V], old[MAX_STREAMS][V];
#pragma unroll
        for (int v = 0; v < V; ++v) y[v] = a.bias ? a.bias[c + v] : 0.f;
        for (int p = 0; p < a.P; ++p) {
            if constexpr (V == 4) {
                const float4 q = *reinterpret_cast<const float4*>(a.sums + p * plane + at);
                y[0] += q.x; y[1] += q.y; y[2] += q.z; y[3] += q.w;
            } else {
                y[0] += a.sums[p * plane + at];
            }
        }
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) {
            if (s >= a.S) break;
            if constexpr (V == 4) {
                const float4 q = *reinterpret_cast<const float4*>(a.xs + s * plane + at);
                old[s][0] = q.x; old[s][1] = q.y; old[s][2] = q.z; old[s][3] = q.w;
            } else {
                old[s][0] = a.xs[s * plane + at];
            }
        }
#pragma unroll
        for (int to = 0; to < MAX_STREAMS; ++to) {
            if (to >= a.S) break;
            float out[V];
#pragma unroll
            for (int v = 0; v < V; ++v) out[v] = m[a.S * a.S + to] * y[v];
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s) {
                if (s >= a.S) break;
#pragma unroll
                for (int v = 0; v < V; ++v) out[v] += m[s * a.S + to] * old[s][v];
            }
            if constexpr (V == 4) *reinterpret_cast<float4*>(a.xs + to * plane + at) = (float4){out[0], out[1], out[2], out[3]};
            else a.xs[to * plane + at] = out[0];
        }
    }
}

// A write and the next read with its RMS norm: one block a row.  The row of the next branch's input is kept in LDS between
// the sum of squares and the store; the new values of a column are summed in the order of the streams, as the read
// kernel sums them, so the result is the same number as from a write and a read.
struct StreamsWriteReadArgs {
    StreamsWriteArgs w;
    const float* w_in;     // [S] of the read that follows, or null: the plain sum
    const float* norm_w;   // [d]
    float eps;
    elem_t* out;           // [T, d]
};

template <int V>
__global__ __launch_bounds__(256) void streams_write_read_kernel(StreamsWriteReadArgs q) {
    const StreamsWriteArgs& a = q.w;
    __shared__ float m[MAX_STREAMS * MAX_STREAMS + 2 * MAX_STREAMS];
    __shared__ float scratch[4];
    extern __shared__ float row[];  // d floats
    const int SS = a.S * a.S;
    for (int i = threadIdx.x; i < SS + 2 * a.S; i += 256)
        m[i] = i < SS ? a.mix[i] : i < SS + a.S ? a.w_out[i - SS] : (q.w_in ? q.w_in[i - SS - a.S] : 1.0f);
    __syncthreads();
    const int t = blockIdx.x;
    const size_t plane = (size_t)a.T * a.d;
    float ss = 0.f;
    for (int c = threadIdx.x * V; c < a.d; c += 256 * V) {
        const size_t at = (size_t)t * a.d + c;
        float y[V], old[MAX_STREAMS][V], u[V];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            y[v] = a.bias ? a.bias[c + v] : 0.f;
            u[v] = 0.f;
        }
        for (int p = 0; p < a.P; ++p) {
            if constexpr (V == 4) {
                const float4 z = *reinterpret_cast<const float4*>(a.sums + p * plane + at);
                y[0] += z.x; y[1] += z.y; y[2] += z.z; y[3] += z.w;
            } else {
                y[0] += a.sums[p * plane + at];
            }
        }
#pragma unroll
        for (int s = 0; s < MAX_STREAMS; ++s) {
            if (s >= a.S) break;
            if constexpr (V == 4) {
                const float4 z = *reinterpret_cast<const float4*>(a.xs + s * plane + at);
                old[s][0] = z.x; old[s][1] = z.y; old[s][2] = z.z; old[s][3] = z.w;
            } else {
                old[s][0] = a.xs[s * plane + at];
            }
        }
#pragma unroll
        for (int to = 0; to < MAX_STREAMS; ++to) {
            if (to >= a.S) break;
            float out[V];
#pragma unroll
            for (int v = 0; v < V; ++v) out[v] = m[SS + to] * y[v];
#pragma unroll
            for (int s = 0; s < MAX_STREAMS; ++s) {
                if (s >= a.S) break;
#pragma unroll
                for (int v = 0; v < V; ++v) out[v] += m[s * a.S + to] * old[s][v];
            }
            if constexpr (V == 4) *reinterpret_cast<float4*>(a.xs + to * plane + at) = (float4){out[0], out[1], out[2], out[3]};
            else a.xs[to * plane + at] = out[0];
#pragma unroll
            for (int v = 0; v < V; ++v) u[v] += m[SS + a.S + to] * out[v];
        }
#pragma unroll
        for (int v = 0; v < V; ++v) {
            row[c + v] = u[v];
            ss += u[v] * u[v];
        }
    }
    ss = block_sum<256>(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)a.d + q.eps);
    for (int c = threadIdx.x; c < a.d; c += 256) q.out[(size_t)t * a.d + c] = from_f32<elem_t>(row[c] * inv * q.norm_w[c]);
}

}  // namespace ms

using namespace ms;

constexpr int STREAMS_MAX_ROW = 15000;
extern "C" int ms_streams_max() { return MAX_STREAMS; }
extern "C" int ms_streams_max_row() { return STREAMS_MAX_ROW; }

// rows null: every row.  norm_w null: the sum itself, 32-bit, into out_f32; else its RMS norm in the element type into out.
extern "C" int ms_streams_read(const float* xs, const float* w_in, const int* rows, int R, const float* norm_w, float eps, float* out_f32,
                               void* out, int S, int T, int d, hipStream_t stream) {
    MS_REQUIRE(S >= 1 && S <= MAX_STREAMS && T > 0 && d > 0 && R > 0, "streams_read: %d streams (at most %d) of %d rows of %d, %d rows read", S,
               MAX_STREAMS, T, d, R);
    MS_REQUIRE(rows || R == T, "streams_read: %d rows of %d without a list of rows", R, T);
    StreamsReadArgs a{xs, w_in, rows, norm_w, eps, out_f32, (elem_t*)out, S, T, d};
    if (norm_w) {
        MS_REQUIRE(d <= STREAMS_MAX_ROW && out, "streams_read: a normed row of %d numbers (at most %d)", d, STREAMS_MAX_ROW);
        hipLaunchKernelGGL(streams_read_kernel<true>, dim3(R), dim3(256), (size_t)d * sizeof(float), stream, a);
    } else {
        MS_REQUIRE(out_f32, "streams_read: no output");
        hipLaunchKernelGGL(streams_read_kernel<false>, dim3(R), dim3(256), 0, stream, a);
    }
    return check_launch("streams_read");
}

extern "C" int ms_streams_write(float* xs, const float* sums, int P, const float* bias, const float* mix, const float* w_out, int S, int T,
                                int d, hipStream_t stream) {
    MS_REQUIRE(S >= 1 && S <= MAX_STREAMS && T > 0 && d > 0 && P >= 1, "streams_write: %d streams (at most %d) of %d rows of %d, %d sums", S,
               MAX_STREAMS, T, d, P);
    StreamsWriteArgs a{xs, sums, bias, mix, w_out, P, S, T, d};
    const long n = (long)T * d;
    if (d % 4 == 0) hipLaunchKernelGGL(streams_write_kernel<4>, dim3((unsigned)std::min<long>(ceil_div(n / 4, 256L), 65535L * 16)), dim3(256), 0, stream, a);
    else hipLaunchKernelGGL(streams_write_kernel<1>, dim3((unsigned)std::min<long>(ceil_div(n, 256L), 65535L * 16)), dim3(256), 0, stream, a);
    return check_launch("streams_write");
}

// The write above and, in the same kernel, the read of the branch that follows: out = rmsnorm(sum_s w_in[s] xs'[s]) * norm_w
// in the element type, from the streams as they are written.
extern "C" int ms_streams_write_read(float* xs, const float* sums, int P, const float* bias, const float* mix, const float* w_out,
                                     const float* w_in, const float* norm_w, float eps, void* out, int S, int T, int d, hipStream_t stream) {
    MS_REQUIRE(S >= 1 && S <= MAX_STREAMS && T > 0 && d > 0 && P >= 1, "streams_write_read: %d streams (at most %d) of %d rows of %d, %d sums", S,
               MAX_STREAMS, T, d, P);
    MS_REQUIRE(d <= STREAMS_MAX_ROW && norm_w && out, "streams_write_read: a normed row of %d numbers (at most %d)", d, STREAMS_MAX_ROW);
    StreamsWriteReadArgs q{{xs, sums, bias, mix, w_out, P, S, T, d}, w_in, norm_w, eps, (elem_t*)out};
    if (d % 4 == 0) hipLaunchKernelGGL(streams_write_read_kernel<4>, dim3(T), dim3(256), (size_t)d * sizeof(float), stream, q);
    else hipLaunchKernelGGL(streams_write_read_kernel<1>, dim3(T), dim3(256), (size_t)d * sizeof(float), stream, q);
    return check_launch("streams_write_read");
}
