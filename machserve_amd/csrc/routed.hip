// A feed-forward of many small experts of which a token uses a few: the router, and the experts' activation.
//
// The router's logits are 32-bit sums of 32-bit weights times the rows as the feed-forward's products read them (in the
// element type, which the 32-bit build does not round); a row's `top` largest logits choose its experts (the lower
// index wins a tie), and their weights are the softmax over the chosen logits alone.  The experts' up projections are one
// matrix [experts * ff (+ shared), width] and their down projections one matrix [width, experts * ff (+ shared)], so the
// weighted sum of the chosen experts' outputs is ONE product over activations in which an expert's columns are
// act(up) * (the row's weight for that expert), zero for an expert the row did not choose, and the columns of an
// expert that every row uses (beyond experts * ff) carry weight one.  Nothing here depends on what else is in the step.
//
// A second way to score (`softmax_all`): the scores are the softmax over every router output, the choice is by score plus
// a correction per output, and the weights are the chosen scores over their sum (+ 1e-20).  Gated experts
// act(gate) * up: the gates of all experts are the first half of the up product's columns.  Router outputs beyond the
// experts stand for experts that return their input: `add_scaled_rows` adds the input's rows with those weights.
#include "common.cuh"

namespace ms {

constexpr int MAX_EXPERTS = 1024;

// gates[t, e] = the row's weight for expert e, 0 where it was not chosen.  One block a row: a wave a logit in turn.
__global__ __launch_bounds__(256) void route_kernel(const elem_t* __restrict__ x, const float* __restrict__ w,
                                                    const float* __restrict__ bias, float* __restrict__ gates, int d, int E, int top,
                                                    int softmax_all, const float* __restrict__ correction) {
    __shared__ float z[MAX_EXPERTS];
    __shared__ float score[MAX_EXPERTS];
    __shared__ float chosen_z[64];
    __shared__ int chosen_e[64];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const elem_t* row = x + (size_t)t * d;
    for (int e = wave; e < E; e += 4) {
        const float* we = w + (size_t)e * d;
        float acc = 0.f;
#pragma unroll 8
        for (int c = lane; c < d; c += 64) acc += to_f32(row[c]) * we[c];
        acc = wave_sum(acc);
        if (lane == 0) z[e] = acc + (bias ? bias[e] : 0.f);
    }
    __syncthreads();
    if (wave == 0 && softmax_all) {
        // scores over every output; what is compared below is the score plus the correction
        float m = -INFINITY;
        for (int e = lane; e < E; e += 64) m = fmaxf(m, z[e]);
        m = wave_max(m);
        float sum = 0.f;
        for (int e = lane; e < E; e += 64) sum += expf(z[e] - m);
        sum = wave_sum(sum);
        for (int e = lane; e < E; e += 64) {
            const float sc = expf(z[e] - m) / sum;
            score[e] = sc;
            z[e] = sc + (correction ? correction[e] : 0.f);
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (wave == 0) {
        // `top` rounds of a maximum over the wave; the winner leaves the list
        for (int k = 0; k < top; ++k) {
            float best = -INFINITY;
            int at = MAX_EXPERTS;
            for (int e = lane; e < E; e += 64)
                if (z[e] > best) { best = z[e]; at = e; }
            for (int o = 32; o > 0; o >>= 1) {
                const float ob = __shfl_xor(best, o, WAVE);
                const int oa = __shfl_xor(at, o, WAVE);
                if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
            }
            if (lane == 0) {
                chosen_z[k] = best;
                chosen_e[k] = at;
                if (at < E) z[at] = -INFINITY;
            }
            __builtin_amdgcn_wave_barrier();
            __threadfence_block();
        }
    }
    __syncthreads();
    float* g = gates + (size_t)t * E;
    for (int e = threadIdx.x; e < E; e += 256) g[e] = 0.f;
    __syncthreads();
    if (threadIdx.x == 0 && softmax_all) {
        float sum = 0.f;
        for (int k = 0; k < top; ++k)
            if (chosen_e[k] < E) sum += score[chosen_e[k]];
        for (int k = 0; k < top; ++k)
            if (chosen_e[k] < E) g[chosen_e[k]] = score[chosen_e[k]] / (sum + 1e-20f);
    } else if (threadIdx.x == 0) {
        const float m = chosen_z[0];  // the first chosen is the largest
        float sum = 0.f;
        for (int k = 0; k < top; ++k) sum += expf(chosen_z[k] - m);
        for (int k = 0; k < top; ++k)
            if (chosen_e[k] < E) g[chosen_e[k]] = expf(chosen_z[k] - m) / sum;
    }
}

// act: 0 the exact GELU (erf), 1 its tanh form, 2 SiLU
__device__ __forceinline__ float expert_activation(float z, int act) {
    if (act == 0) return 0.5f * z * (1.0f + erff(z * 0.7071067811865476f));
    if (act == 1) return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    return z / (1.0f + expf(-z));
}

// a[t, c] = act(up[t, c]) * gates[t, c / ff] for c < E * ff, act(up[t, c]) beyond (experts that every row uses)
constexpr int ACT_COLS = 2048;  // columns of a row that a block takes
template <int V>  // columns a thread takes at once: 4 where an expert's columns and the row are multiples of four
__global__ __launch_bounds__(256) void expert_act_kernel(const float* __restrict__ up, const float* __restrict__ gates,
                                                         elem_t* __restrict__ out, int n, int E, int ff, int act, int ld_gates, int gated) {
    const int t = blockIdx.x, c0 = blockIdx.y * ACT_COLS, c1 = min(n, c0 + ACT_COLS);
    const float* g = gates + (size_t)t * ld_gates;
    if (gated) {  // up [T, 2 n]: the gates' columns, then the up projections'
        const float* row = up + (size_t)t * 2 * n;
#pragma unroll 2
        for (int c = c0 + threadIdx.x * V; c < c1; c += 256 * V) {
            const int e = c / ff;  // V columns lie in one expert (ff is a multiple of V)
            const float w = e < E ? g[e] : 1.0f;
            elem_t* o = out + (size_t)t * n + c;
            if constexpr (V == 4) {
                float4 a = (float4){0.f, 0.f, 0.f, 0.f}, b = a;
                if (w != 0.f) {
                    a = *reinterpret_cast<const float4*>(row + c);
                    b = *reinterpret_cast<const float4*>(row + n + c);
                }
                o[0] = from_f32<elem_t>(w != 0.f ? expert_activation(a.x, act) * b.x * w : 0.f);
                o[1] = from_f32<elem_t>(w != 0.f ? expert_activation(a.y, act) * b.y * w : 0.f);
                o[2] = from_f32<elem_t>(w != 0.f ? expert_activation(a.z, act) * b.z * w : 0.f);
                o[3] = from_f32<elem_t>(w != 0.f ? expert_activation(a.w, act) * b.w * w : 0.f);
            } else {
                o[0] = from_f32<elem_t>(w != 0.f ? expert_activation(row[c], act) * row[n + c] * w : 0.f);
            }
        }
        return;
    }
#pragma unroll 2
    for (int c = c0 + threadIdx.x * V; c < c1; c += 256 * V) {
        const int e = c / ff;
        const float w = e < E ? g[e] : 1.0f;
        // an expert the row did not choose contributes an exact zero, whatever its product holds
        if constexpr (V == 4) {
            float4 v = (float4){0.f, 0.f, 0.f, 0.f};
            if (w != 0.f) v = *reinterpret_cast<const float4*>(up + (size_t)t * n + c);
            elem_t* o = out + (size_t)t * n + c;
            o[0] = from_f32<elem_t>(w != 0.f ? expert_activation(v.x, act) * w : 0.f);
            o[1] = from_f32<elem_t>(w != 0.f ? expert_activation(v.y, act) * w : 0.f);
            o[2] = from_f32<elem_t>(w != 0.f ? expert_activation(v.z, act) * w : 0.f);
            o[3] = from_f32<elem_t>(w != 0.f ? expert_activation(v.w, act) * w : 0.f);
        } else {
            out[(size_t)t * n + c] = from_f32<elem_t>(w != 0.f ? expert_activation(up[(size_t)t * n + c], act) * w : 0.f);
        }
    }
}

// x[t, c] += (sum of weights[t, first .. first + count]) * h[t, c]: rows of a part's input added with a weight a row
__global__ __launch_bounds__(256) void add_scaled_rows_kernel(float* __restrict__ x, const elem_t* __restrict__ h,
                                                              const float* __restrict__ weights, int ld_w, int first, int count, int d) {
    const int t = blockIdx.x;
    float w = 0.f;
    for (int i = 0; i < count; ++i) w += weights[(size_t)t * ld_w + first + i];
    if (w == 0.f) return;
    for (int c = blockIdx.y * 1024 + threadIdx.x; c < min(d, (int)(blockIdx.y + 1) * 1024); c += 256)
        x[(size_t)t * d + c] += w * to_f32(h[(size_t)t * d + c]);
}

}  // namespace ms

using namespace ms;

extern "C" int ms_route_max_experts() { return MAX_EXPERTS; }

extern "C" int ms_route(const void* x, const float* w, const float* bias, float* gates, int T, int d, int E, int top, int softmax_all,
                        const float* correction, hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0 && E > 0 && E <= MAX_EXPERTS, "route: %d rows of %d over %d experts (at most %d)", T, d, E, MAX_EXPERTS);
    MS_REQUIRE(top >= 1 && top <= E && top <= 64, "route: %d of %d experts a row (at most 64)", top, E);
    hipLaunchKernelGGL(route_kernel, dim3(T), dim3(256), 0, stream, (const elem_t*)x, w, bias, gates, d, E, top, softmax_all, correction);
    return check_launch("route");
}

// n: columns of the output; with `gated`, up has 2 n columns.  ld_gates: numbers a row of gates has (>= E).
extern "C" int ms_expert_act(const float* up, const float* gates, void* out, int T, int n, int E, int ff, int act, int ld_gates, int gated,
                             hipStream_t stream) {
    MS_REQUIRE(T > 0 && n > 0 && E >= 0 && ff > 0 && (long)E * ff <= n && ld_gates >= E, "expert_act: %d columns for %d experts of %d", n, E, ff);
    MS_REQUIRE(act >= 0 && act <= 2, "expert_act: activation %d", act);
    const dim3 grid(T, ceil_div(n, ACT_COLS));
    if (n % 4 == 0 && ff % 4 == 0) hipLaunchKernelGGL(expert_act_kernel<4>, grid, dim3(256), 0, stream, up, gates, (elem_t*)out, n, E, ff, act, ld_gates, gated);
    else hipLaunchKernelGGL(expert_act_kernel<1>, grid, dim3(256), 0, stream, up, gates, (elem_t*)out, n, E, ff, act, ld_gates, gated);
    return check_launch("expert_act");
}

extern "C" int ms_add_scaled_rows(float* x, const void* h, const float* weights, int ld_w, int first, int count, int T, int d,
                                  hipStream_t stream) {
    MS_REQUIRE(T > 0 && d > 0 && first >= 0 && count >= 1 && first + count <= ld_w, "add_scaled_rows: weights %d .. %d of %d", first,
               first + count, ld_w);
    hipLaunchKernelGGL(add_scaled_rows_kernel, dim3(T, ceil_div(d, 1024)), dim3(256), 0, stream, x, (const elem_t*)h, weights, ld_w, first,
                       count, d);
    return check_launch("add_scaled_rows");
}
