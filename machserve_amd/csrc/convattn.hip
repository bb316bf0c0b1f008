// What grouped-query attention with a short convolution behind its projections needs around the paged attention
// kernels: one row kernel that finishes a row of the fused projection [q | k | gate] from its 32-bit partial sums,
// and the kernel that brings the convolution's state up to date.
//
// Per row: a causal convolution over time on every channel of q and k (the inputs before the step's first row of the
// request come from the request's state, the last taps - 1 projected rows; before the request's start they are
// zero); the values are the convolved keys as they are; q and k of every head are divided by their root mean square
// (no weight); q is multiplied by a temperature that grows with the position,
// 1 + coef * ln(floor((p + 1) / every) + 1); the gate's columns go through a sigmoid and are left as 32-bit
// factors, one per (row, head), that the attention kernel applies to its output.  Keys and values are written into
// the row's page, filled with zeros up to the attention tile's head size (the pools start as zeros; q's filling is
// written).  Everything here is 32-bit; the element type is what q and the pages store.
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

struct ConvRowArgs {
    const float* proj;      // [n_partials, T, stride]: q [H, d], k [KV, d], gate [H] (gate only if gate_out)
    int n_partials;
    size_t partial_stride;
    int stride;
    const float* conv_w;    // [(H + KV) * d, taps] or null: no convolution
    int taps;
    const float* state;     // [slots, taps - 1, (H + KV) * d], oldest first
    const int* seq_q_start;
    const int* seq_slot;
    int S;
    const int* positions;   // [T]
    int unit_norm;          // q and k of a head divided by their root mean square
    float eps;
    float temp_coef;        // 0: no temperature
    int temp_every;
    int values_are_keys;    // the value pool receives the keys before their norm
    const int* slot_map;    // [T]
    elem_t* q_out;          // [T, H, dp]
    elem_t* kpool;          // [pages, KV, ps, dp]
    elem_t* vpool;          // [pages, KV, dp, ps]
    float* gate_out;        // [T, H] or null
    int H, KV, d, dp, ps;
};

__global__ __launch_bounds__(256) void conv_row_kernel(ConvRowArgs a) {
    extern __shared__ float row[];  // (H + KV) * d floats: the convolved row
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int nq = a.H * a.d, C = (a.H + a.KV) * a.d;
    const int s = seq_of_row(t, a.seq_q_start, a.S);
    const int j = t - a.seq_q_start[s];
    const int keep = a.taps - 1;
    const float* st = keep > 0 ? a.state + (size_t)a.seq_slot[s] * keep * C : nullptr;
    auto projected = [&](int r, int c) {
        float v = 0.f;
#pragma unroll 8
        for (int p = 0; p < a.n_partials; ++p) v += a.proj[p * a.partial_stride + (size_t)r * a.stride + c];  // eight loads in flight
        return v;
    };
    for (int c = threadIdx.x; c < C; c += 256) {
        float y;
        if (a.conv_w) {
            y = 0.f;
            for (int k = 0; k < a.taps; ++k) {
                const int back = keep - k, idx = j - back;
                const float u = idx >= 0 ? projected(t - back, c) : st[(size_t)(keep + idx) * C + c];
                y += a.conv_w[(size_t)c * a.taps + k] * u;
            }
        } else {
            y = projected(t, c);
        }
        row[c] = y;
    }
    if (a.gate_out)
        for (int h = threadIdx.x; h < a.H; h += 256) a.gate_out[(size_t)t * a.H + h] = 1.0f / (1.0f + expf(-projected(t, C + h)));
    __syncthreads();
    const int pos = a.positions[t];
    float temp = 1.0f;
    if (a.temp_coef != 0.f) temp = 1.0f + a.temp_coef * logf((float)((pos + 1) / a.temp_every) + 1.0f);
    const int slot = a.slot_map[t];
    const int page = slot >= 0 ? slot / a.ps : 0, off = slot >= 0 ? slot % a.ps : 0;
    // a wave a head: q heads first, then k heads
    for (int hh = wave; hh < a.H + a.KV; hh += 4) {
        const float* head = row + hh * a.d;
        float ss = 0.f;
        for (int e = lane; e < a.d; e += 64) ss += head[e] * head[e];
        ss = wave_sum(ss);
        const float inv = a.unit_norm ? 1.0f / sqrtf(ss / (float)a.d + a.eps) : 1.0f;
        if (hh < a.H) {
            elem_t* dst = a.q_out + ((size_t)t * a.H + hh) * a.dp;
            for (int e = lane; e < a.dp; e += 64) dst[e] = from_f32<elem_t>(e < a.d ? head[e] * inv * temp : 0.f);
        } else if (slot >= 0) {
            const int kh = hh - a.H;
            elem_t* krow = a.kpool + (((size_t)page * a.KV + kh) * a.ps + off) * a.dp;
            elem_t* vcol = a.vpool + ((size_t)page * a.KV + kh) * a.dp * a.ps + off;
            for (int e = lane; e < a.d; e += 64) {
                krow[e] = from_f32<elem_t>(head[e] * inv);
                if (a.values_are_keys) vcol[(size_t)e * a.ps] = from_f32<elem_t>(head[e]);
            }
        }
    }
}

// The same with a wave a head and R consecutive rows of the step a block, for up to FAST_TAPS taps and heads of up to
// 256 numbers: a lane holds its channels' projected rows t0 - (taps - 1) .. t0 + R - 1 in registers (each row of the
// projection is read (R + taps - 1) / R times instead of `taps` times), all loads of a chunk are asked for before the
// first is used, and a head's sum of squares is a reduction over the wave: no LDS and no barrier.  R = 8 in steps of
// many rows, 1 where rows are few (decoding: the blocks would not fill the chip otherwise, and a row's earlier inputs
// come from its request's state anyway).  The gate's columns are one more "head".  Same sums in the same order as the
// kernel above.
constexpr int FAST_TAPS = 8, FAST_CHUNKS = 4;

// A head of a row that is the first of its request in this step (decoding): every earlier input comes from the state.
// All loads (eight partial sums at a time, the state's rows, the taps' weights, for every chunk of the head) are asked
// for on one straight path from clamped addresses and picked afterwards, so the wave waits for memory once instead of
// once a load (a load under a condition makes every later wait a wait for everything).
__device__ __forceinline__ void conv_head_first_row(const ConvRowArgs& a, int t, int hh, int lane, int slot_of_state, int pos, int slot) {
    const int n_heads = a.H + a.KV, C = n_heads * a.d, keep = a.taps - 1;
    const float* st = keep > 0 ? a.state + (size_t)slot_of_state * keep * C : a.proj;
    const float* row = a.proj + (size_t)t * a.stride;
    float y[FAST_CHUNKS];
    float pr[FAST_CHUNKS][8], sv[FAST_CHUNKS][FAST_TAPS - 1], wv[FAST_CHUNKS][FAST_TAPS];
#pragma unroll
    for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
        const int c = hh * a.d + min(lane + 64 * ci, a.d - 1);
#pragma unroll
        for (int p = 0; p < 8; ++p) pr[ci][p] = row[(size_t)min(p, a.n_partials - 1) * a.partial_stride + c];
#pragma unroll
        for (int k = 0; k < FAST_TAPS - 1; ++k) sv[ci][k] = st[(size_t)min(k, max(keep - 1, 0)) * C + c];
#pragma unroll
        for (int k = 0; k < FAST_TAPS; ++k) wv[ci][k] = a.conv_w ? a.conv_w[(size_t)c * a.taps + min(k, keep)] : 1.0f;
    }
#pragma unroll
    for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
        const int c = hh * a.d + min(lane + 64 * ci, a.d - 1);
        float u = 0.f;
#pragma unroll
        for (int p = 0; p < 8; ++p) u += p < a.n_partials ? pr[ci][p] : 0.f;
        for (int p = 8; p < a.n_partials; ++p) u += row[(size_t)p * a.partial_stride + c];
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < FAST_TAPS - 1; ++k) acc += k < keep ? wv[ci][k] * sv[ci][k] : 0.f;
#pragma unroll
        for (int k = 0; k < FAST_TAPS; ++k) acc += k == keep ? wv[ci][k] * u : 0.f;
        y[ci] = lane + 64 * ci < a.d ? acc : 0.f;
    }
    float ss = 0.f;
#pragma unroll
    for (int ci = 0; ci < FAST_CHUNKS; ++ci) ss += y[ci] * y[ci];
    ss = wave_sum(ss);
    const float inv = a.unit_norm ? 1.0f / sqrtf(ss / (float)a.d + a.eps) : 1.0f;
    if (hh < a.H) {
        float temp = 1.0f;
        if (a.temp_coef != 0.f) temp = 1.0f + a.temp_coef * logf((float)((pos + 1) / a.temp_every) + 1.0f);
        elem_t* dst = a.q_out + ((size_t)t * a.H + hh) * a.dp;
#pragma unroll
        for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
            const int e = lane + 64 * ci;
            if (e < a.dp) dst[e] = from_f32<elem_t>(e < a.d ? y[ci] * inv * temp : 0.f);
        }
    } else if (slot >= 0) {
        const int page = slot / a.ps, off = slot % a.ps, kh = hh - a.H;
        elem_t* krow = a.kpool + (((size_t)page * a.KV + kh) * a.ps + off) * a.dp;
        elem_t* vcol = a.vpool + ((size_t)page * a.KV + kh) * a.dp * a.ps + off;
#pragma unroll
        for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
            const int e = lane + 64 * ci;
            if (e < a.d) {
                krow[e] = from_f32<elem_t>(y[ci] * inv);
                if (a.values_are_keys) vcol[(size_t)e * a.ps] = from_f32<elem_t>(y[ci]);
            }
        }
    }
}

template <int R>
__global__ __launch_bounds__(256) void conv_head_kernel(ConvRowArgs a, int T) {
    constexpr int W = R + FAST_TAPS - 1;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int hh = blockIdx.y * 4 + wave, t0 = blockIdx.x * R;
    const int n_heads = a.H + a.KV;
    if (hh > n_heads || (hh == n_heads && !a.gate_out)) return;  // the same for the whole wave; the kernel has no barrier
    const int C = n_heads * a.d;
    auto projected = [&](int r, int c) {
        float v = 0.f;
#pragma unroll 8
        for (int p = 0; p < a.n_partials; ++p) v += a.proj[p * a.partial_stride + (size_t)r * a.stride + c];  // eight loads in flight
        return v;
    };
    if (hh == n_heads) {
        for (int i = 0; i < R; ++i) {
            const int t = t0 + i;
            if (t >= T) break;
            for (int h = lane; h < a.H; h += 64) a.gate_out[(size_t)t * a.H + h] = 1.0f / (1.0f + expf(-projected(t, C + h)));
        }
        return;
    }
    const int keep = a.taps - 1;
    if constexpr (R == 1) {
        // every request of the step has one row, so row t is request t and its first row in this step
        if (a.S == T && a.seq_q_start[t0] == t0) {
            conv_head_first_row(a, t0, hh, lane, a.seq_slot[t0], a.positions[t0], a.slot_map[t0]);
            return;
        }
    }
    // per row of the block: how many rows of its request the step holds before it, and the request's state
    // (where every request of the step has one row, row t is request t, which two loads side by side confirm: no search
    // with its chain of trips to memory; the row's position and address are asked for here, long before they are used)
    int before[R], pos[R], slot[R];
    const float* st[R];
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int t = min(t0 + i, T - 1);
        int s = min(t, a.S - 1);
        if (!(a.S == T && a.seq_q_start[s] == t && (s == a.S - 1 || a.seq_q_start[s + 1] > t))) s = seq_of_row(t, a.seq_q_start, a.S);
        before[i] = t - a.seq_q_start[s];
        st[i] = keep > 0 ? a.state + (size_t)a.seq_slot[s] * keep * C : nullptr;
        pos[i] = a.positions[t];
        slot[i] = a.slot_map[t];
    }
    float y[FAST_CHUNKS][R];
#pragma unroll
    for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
        const int e = lane + 64 * ci;
        const bool live = e < a.d;  // the same for the wave's later chunks too: they are skipped whole
        if (ci * 64 >= a.d) {
#pragma unroll
            for (int i = 0; i < R; ++i) y[ci][i] = 0.f;
            continue;
        }
        const int c = hh * a.d + (live ? e : 0);
        float win[W], cw[FAST_TAPS];
#pragma unroll
        for (int w = 0; w < W; ++w) {
            const int r = t0 - keep + w;
            win[w] = (w < R + keep && r >= 0 && r < T) ? projected(r, c) : 0.f;
        }
#pragma unroll
        for (int k = 0; k < FAST_TAPS; ++k) cw[k] = k < a.taps ? (a.conv_w ? a.conv_w[(size_t)c * a.taps + k] : 1.0f) : 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            float acc = 0.f;
#pragma unroll
            for (int k = 0; k < FAST_TAPS; ++k) {
                if (k < a.taps) {
                    // tap k reads the row (taps - 1 - k) back: of this step if the request has that many rows before, else of its state
                    const float u = k >= keep - before[i] ? win[i + k] : st[i][(size_t)(before[i] + k) * C + c];
                    acc += cw[k] * u;
                }
            }
            y[ci][i] = live ? acc : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < R; ++i) {
        const int t = t0 + i;
        if (t >= T) break;
        float ss = 0.f;
#pragma unroll
        for (int ci = 0; ci < FAST_CHUNKS; ++ci) ss += y[ci][i] * y[ci][i];
        ss = wave_sum(ss);
        const float inv = a.unit_norm ? 1.0f / sqrtf(ss / (float)a.d + a.eps) : 1.0f;
        if (hh < a.H) {
            float temp = 1.0f;
            if (a.temp_coef != 0.f) temp = 1.0f + a.temp_coef * logf((float)((pos[i] + 1) / a.temp_every) + 1.0f);
            elem_t* dst = a.q_out + ((size_t)t * a.H + hh) * a.dp;
#pragma unroll
            for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
                const int e = lane + 64 * ci;
                if (e < a.dp) dst[e] = from_f32<elem_t>(e < a.d ? y[ci][i] * inv * temp : 0.f);
            }
        } else {
            if (slot[i] < 0) continue;
            const int page = slot[i] / a.ps, off = slot[i] % a.ps, kh = hh - a.H;
            elem_t* krow = a.kpool + (((size_t)page * a.KV + kh) * a.ps + off) * a.dp;
            elem_t* vcol = a.vpool + ((size_t)page * a.KV + kh) * a.dp * a.ps + off;
#pragma unroll
            for (int ci = 0; ci < FAST_CHUNKS; ++ci) {
                const int e = lane + 64 * ci;
                if (e < a.d) {
                    krow[e] = from_f32<elem_t>(y[ci][i] * inv);
                    if (a.values_are_keys) vcol[(size_t)e * a.ps] = from_f32<elem_t>(y[ci][i]);
                }
            }
        }
    }
}

// The state after the step: the last taps - 1 projected rows of each request, old ones where the step brought fewer.
constexpr int CONV_MAX_TAPS = 16;
__global__ __launch_bounds__(256) void conv_row_state_kernel(const float* __restrict__ proj, int n_partials, size_t partial_stride, int stride,
                                                             float* __restrict__ state, const int* __restrict__ seq_q_start,
                                                             const int* __restrict__ seq_q_len, const int* __restrict__ seq_slot, int C,
                                                             int taps) {
    const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
    if (c >= C) return;
    const int n = seq_q_len[s], q0 = seq_q_start[s], keep = taps - 1;
    float* st = state + (size_t)seq_slot[s] * keep * C;
    float v[CONV_MAX_TAPS];
    for (int i = 0; i < keep; ++i) {
        const int idx = n - keep + i;  // among the step's rows; negative: an older input
        float u = 0.f;
        if (idx >= 0) {
#pragma unroll 8
            for (int p = 0; p < n_partials; ++p) u += proj[p * partial_stride + (size_t)(q0 + idx) * stride + c];
        } else {
            u = st[(size_t)(keep + idx) * C + c];
        }
        v[i] = u;
    }
    for (int i = 0; i < keep; ++i) st[(size_t)i * C + c] = v[i];
}

// ---- rows of q, k and v that are finished elsewhere (a convolution on all three, say), given as 32-bit numbers ------------
// An RMS norm over the whole of q and one over the whole of k (weights; null: none), then the rotation of the first `rot`
// numbers of every head of q and k by position * inv_freq, pairs (i, i + rot / 2) or neighbours (2i, 2i + 1); q goes out
// in the element type with heads of dp numbers (zeros from d on), k and v into their pages, whose heads are dp wide too
// (what lies beyond d, or beyond dv for a value, is never written and stays zero).
struct FinishArgs {
    const float* rows;      // [T, stride]: q [H, d], k [KV, d], v [KV, dv]
    int stride;
    const float* q_norm;    // [H * d] or null
    const float* k_norm;    // [KV * d] or null
    float eps;
    const int* positions;   // [T]
    const float* inv_freq;  // [rot / 2] or null: no rotation
    int rot, neighbours;
    const int* slot_map;    // [T] page * ps + offset
    elem_t* q_out;          // [T, H * dp]
    elem_t* kpool;          // [pages, KV, ps, dp]
    elem_t* vpool;          // [pages, KV, dp, ps]
    int H, KV, d, dv, dp, ps;
};

__global__ __launch_bounds__(256) void finish_rows_kernel(FinishArgs a) {
    __shared__ float scratch[4];
    extern __shared__ float lds[];
    float* row = lds;                 // stride floats
    float* cs = lds + a.stride;       // rot / 2 cosines, then rot / 2 sines
    const int t = blockIdx.x, nq = a.H * a.d, nk = a.KV * a.d, nv = a.KV * a.dv, half = a.rot / 2;
    float ssq = 0.f, ssk = 0.f;
    for (int c = threadIdx.x; c < nq + nk + nv; c += 256) {
        const float v = a.rows[(size_t)t * a.stride + c];
        row[c] = v;
        if (c < nq) ssq += v * v;
        else if (c < nq + nk) ssk += v * v;
    }
    for (int j = threadIdx.x; j < half; j += 256) {
        float c = 1.f, s = 0.f;
        if (a.inv_freq) sincosf((float)a.positions[t] * a.inv_freq[j], &s, &c);
        cs[j] = c;
        cs[half + j] = s;
    }
    ssq = block_sum<256>(ssq, scratch);
    ssk = block_sum<256>(ssk, scratch);
    const float inv_q = a.q_norm ? 1.0f / sqrtf(ssq / (float)nq + a.eps) : 1.0f;
    const float inv_k = a.k_norm ? 1.0f / sqrtf(ssk / (float)nk + a.eps) : 1.0f;
    __syncthreads();
    const int slot = a.slot_map[t];
    const int page = slot >= 0 ? slot / a.ps : 0, off = slot >= 0 ? slot % a.ps : 0;
    const int fill = a.dp - a.d;
    for (int c = threadIdx.x; c < nq + nk; c += 256) {
        const bool is_q = c < nq;
        const int cc = is_q ? c : c - nq;
        const int h = cc / a.d, i = cc - h * a.d;
        const float inv = is_q ? inv_q : inv_k;
        const float* nw = is_q ? a.q_norm : a.k_norm;
        const float* base = row + (is_q ? 0 : nq) + h * a.d;
        auto normed = [&](int e) { return base[e] * inv * (nw ? nw[h * a.d + e] : 1.0f); };
        float v;
        if (i >= a.rot) {
            v = normed(i);
        } else if (a.neighbours) {
            const int pr = i >> 1;
            v = (i & 1) ? normed(i) * cs[pr] + normed(i - 1) * cs[half + pr] : normed(i) * cs[pr] - normed(i + 1) * cs[half + pr];
        } else {
            v = i < half ? normed(i) * cs[i] - normed(i + half) * cs[half + i] : normed(i) * cs[i - half] + normed(i - half) * cs[i];
        }
        if (is_q) a.q_out[((size_t)t * a.H + h) * a.dp + i] = from_f32<elem_t>(v);
        else if (slot >= 0) a.kpool[(((size_t)page * a.KV + h) * a.ps + off) * a.dp + i] = from_f32<elem_t>(v);
    }
    for (int c = threadIdx.x; c < a.H * fill; c += 256)  // the queries' heads are filled up with zeros
        a.q_out[((size_t)t * a.H + c / fill) * a.dp + a.d + c % fill] = from_f32<elem_t>(0.f);
    for (int c = threadIdx.x; c < nv; c += 256) {
        const int h = c / a.dv, e = c - h * a.dv;
        if (slot >= 0) a.vpool[(((size_t)page * a.KV + h) * a.dp + e) * a.ps + off] = from_f32<elem_t>(row[nq + nk + c]);
    }
}

// Differential attention behind the attention kernel.  o [T, 2 H maps, dp]: the maps of a key/value head's group lie side
// by side, (key/value head, map, head of the group).  A head's result is map 0 minus lam times map 1 over its first dv
// numbers, divided by its root mean square, times `factor`, times sigmoid(gate); heads side by side in rows of ld_out
// numbers (zeros behind H * dv).  A wave a head.
__global__ __launch_bounds__(256) void diff_combine_kernel(const elem_t* __restrict__ o, const float* __restrict__ gate,
                                                           elem_t* __restrict__ out, float lam, float eps, float factor, int H, int KV,
                                                           int dp, int dv, int ld_out) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, h = blockIdx.y * 4 + (threadIdx.x >> 6);
    if (blockIdx.y == 0)
        for (int c = H * dv + threadIdx.x; c < ld_out; c += 256) out[(size_t)t * ld_out + c] = from_f32<elem_t>(0.f);
    if (h >= H) return;  // the same for the whole wave; no barrier below
    const int per = H / KV, kvh = h / per, in_group = h - kvh * per;
    const elem_t* a1 = o + ((size_t)t * 2 * H + (size_t)(kvh * 2) * per + in_group) * dp;
    const elem_t* a2 = a1 + (size_t)per * dp;
    float ss = 0.f;
    for (int e = lane; e < dv; e += 64) {
        const float v = to_f32(a1[e]) - lam * to_f32(a2[e]);
        ss += v * v;
    }
    ss = wave_sum(ss);
    const float inv = factor / sqrtf(ss / (float)dv + eps);
    for (int e = lane; e < dv; e += 64) {
        const float v = to_f32(a1[e]) - lam * to_f32(a2[e]);
        const float gz = gate[(size_t)t * H * dv + h * dv + e];
        out[(size_t)t * ld_out + h * dv + e] = from_f32<elem_t>(v * inv / (1.0f + expf(-gz)));
    }
}

}  // namespace ms

using namespace ms;

constexpr int CONV_MAX_ROW = 15000;
extern "C" int ms_conv_rows_max_row() { return CONV_MAX_ROW; }
extern "C" int ms_conv_rows_max_taps() { return CONV_MAX_TAPS; }

// proj float [n_partials, T, stride]; conv_w null or float [(H + KV) * d, taps]; state float [slots, taps - 1, (H + KV) * d],
// read here and brought up to date by a second launch; gate_out null or float [T, H].
extern "C" int ms_conv_rows(const float* proj, int n_partials, int stride, const float* conv_w, int taps, float* state,
                            const int* seq_q_start, const int* seq_q_len, const int* seq_slot, int S, const int* positions,
                            int unit_norm, float eps, float temp_coef, int temp_every, int values_are_keys, const int* slot_map,
                            void* q_out, void* kpool, void* vpool, float* gate_out, int T, int H, int KV, int d, int dp, int ps,
                            hipStream_t stream) {
    MS_REQUIRE(T > 0 && S > 0 && n_partials >= 1, "conv rows: %d rows of %d requests, %d partial sums", T, S, n_partials);
    const int C = (H + KV) * d;
    MS_REQUIRE(H > 0 && KV > 0 && d > 0 && dp >= d, "conv rows: %d heads, %d key/value heads, head size %d in %d", H, KV, d, dp);
    MS_REQUIRE(stride >= C + (gate_out ? H : 0) && C <= CONV_MAX_ROW, "conv rows: a row of %d numbers (stride %d, at most %d)", C, stride, CONV_MAX_ROW);
    MS_REQUIRE(!conv_w || (taps >= 1 && taps <= CONV_MAX_TAPS && (state || taps == 1)), "conv rows: %d taps (1 to %d, with a state from 2 on)", taps, CONV_MAX_TAPS);
    MS_REQUIRE(temp_coef == 0.f || temp_every > 0, "conv rows: temperature every %d positions", temp_every);
    ConvRowArgs a{proj, n_partials, (size_t)T * stride, stride, conv_w, conv_w ? taps : 1, state, seq_q_start, seq_slot, S, positions,
                  unit_norm, eps, temp_coef, temp_every, values_are_keys, slot_map, (elem_t*)q_out, (elem_t*)kpool, (elem_t*)vpool,
                  gate_out, H, KV, d, dp, ps};
    if (a.taps <= FAST_TAPS && dp <= 64 * FAST_CHUNKS) {
        const int units = ceil_div(H + KV + (gate_out ? 1 : 0), 4);
        if (T > 64) hipLaunchKernelGGL(conv_head_kernel<8>, dim3(ceil_div(T, 8), units), dim3(256), 0, stream, a, T);
        else hipLaunchKernelGGL(conv_head_kernel<1>, dim3(T, units), dim3(256), 0, stream, a, T);
    } else {
        hipLaunchKernelGGL(conv_row_kernel, dim3(T), dim3(256), (size_t)C * sizeof(float), stream, a);
    }
    int rc = check_launch("conv_rows");
    if (rc || !conv_w || taps < 2) return rc;
    hipLaunchKernelGGL(conv_row_state_kernel, dim3(S, ceil_div(C, 256)), dim3(256), 0, stream, proj, n_partials, (size_t)T * stride, stride,
                       state, seq_q_start, seq_q_len, seq_slot, C, taps);
    return check_launch("conv_rows_state");
}

extern "C" int ms_finish_rows(const float* rows, int stride, const float* q_norm, const float* k_norm, float eps, const int* positions,
                              const float* inv_freq, int rot, int neighbours, const int* slot_map, void* q_out, void* kpool, void* vpool,
                              int T, int H, int KV, int d, int dv, int dp, int ps, hipStream_t stream) {
    // KV 0: the rows hold queries only (the layer reads another layer's keys and values); nothing is written to the pools
    MS_REQUIRE(T > 0 && H > 0 && KV >= 0 && d > 0 && dv > 0 && dp >= d && dp >= dv, "finish rows: %d rows, %d / %d heads of %d and %d in %d",
               T, H, KV, d, dv, dp);
    const int n = H * d + KV * d + KV * dv;
    MS_REQUIRE(stride >= n && n + rot <= CONV_MAX_ROW, "finish rows: a row of %d numbers (stride %d, at most %d)", n, stride, CONV_MAX_ROW);
    MS_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= d, "finish rows: %d of %d numbers of a head are rotated", rot, d);
    FinishArgs a{rows, stride, q_norm, k_norm, eps, positions, inv_freq, rot, neighbours, slot_map, (elem_t*)q_out, (elem_t*)kpool,
                 (elem_t*)vpool, H, KV, d, dv, dp, ps};
    hipLaunchKernelGGL(finish_rows_kernel, dim3(T), dim3(256), (size_t)(stride + rot) * sizeof(float), stream, a);
    return check_launch("finish_rows");
}

extern "C" int ms_diff_combine(const void* o, const float* gate, void* out, float lam, float eps, float factor, int T, int H, int KV, int dp,
                               int dv, int ld_out, hipStream_t stream) {
    MS_REQUIRE(T > 0 && H > 0 && KV > 0 && H % KV == 0 && dv > 0 && dp >= dv && ld_out >= H * dv, "diff_combine: %d rows, %d / %d heads of %d in %d",
               T, H, KV, dv, dp);
    hipLaunchKernelGGL(diff_combine_kernel, dim3(T, ceil_div(H, 4)), dim3(256), 0, stream, (const elem_t*)o, gate, (elem_t*)out, lam, eps,
                       factor, H, KV, dp, dv, ld_out);
    return check_launch("diff_combine");
}
