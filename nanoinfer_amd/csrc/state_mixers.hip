// Mixers whose memory of the past is a state of fixed size per request, for gfx950: linear attention with one
// decay a head, and the selective scan (a diagonal recurrence per channel whose step sizes, inputs and read-outs
// depend on the token) with its short causal convolution.
//
// Everything that enters a recurrence is float32: the projections come as float32 rows, states live in float32 in
// the cache manager's state slots, exponentials and softplus are the accurate routines.  A step brings, for every
// sequence b, the rows q_start[b] .. q_start[b] + q_len[b] - 1 (consecutive tokens of that sequence) and the slot
// state_slot[b]; a kernel walks a sequence's rows in order and leaves the state as it is after the last one.
// Every entry point returns 0 or a hipError_t.
#include "common.h"

#include <algorithm>

static inline unsigned blocks_of(size_t n, unsigned per) { return static_cast<unsigned>((n + per - 1) / per); }

__device__ __forceinline__ float silu_f(float z) { return z / (1.0f + expf(-z)); }
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float softplus_f(float z) { return z > 20.f ? z : log1pf(expf(z)); }

// sum over `parts` neighbouring lanes (a power of two), every one of them gets it
__device__ __forceinline__ float parts_sum(float v, int parts) {
    for (int off = 1; off < parts; off <<= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

// ---------------------------------------------------------------- silu of the first n columns of every row
__global__ void silu_rows_kernel(const float* __restrict__ in, int in_stride, float* __restrict__ out, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t t = i / n;
    const int c = static_cast<int>(i % n);
    out[i] = silu_f(in[t * in_stride + c]);
}

NI_EXPORT int ni_silu_rows(const void* in, int in_stride, void* out, int T, int n, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * n;
    if (total == 0) return 0;
    if (in_stride < n) return -1;
    silu_rows_kernel<<<blocks_of(total, 256), 256, 0, stream>>>((const float*)in, in_stride, (float*)out, n, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- linear attention with a decay a head
//   S <- decay[h] S + k v^T,   o = S^T q          S [dk, dv] per head, float32
// act float32 [T, 2 H dk + H dv]: q | k | v (after their activation), head by head.  The state of a slot is
// [H][dv][dkp] (a value channel's column of key channels lies together), dkp = parts * 8 >= dk, the padding zero.
// A column is held by `parts` neighbouring lanes with eight key channels each; a wavefront takes 64 / parts
// columns, a workgroup of four wavefronts four times that.  The next token's operands are asked for before this
// token's arithmetic.
#define DKPT 8

struct DecayOperands {
    float q[DKPT], k[DKPT], v;
};

// `raw`: the row holds the projections themselves and silu is applied here (steps of few tokens, which save a launch so)
__device__ __forceinline__ void decay_load(DecayOperands& o, const float* __restrict__ row, int q_off, int k_off, int v_off,
                                           int ch, int dk, bool whole, bool raw = false) {
    if (whole) {
        const float4 a = *reinterpret_cast<const float4*>(row + q_off + ch), b = *reinterpret_cast<const float4*>(row + q_off + ch + 4);
        const float4 c = *reinterpret_cast<const float4*>(row + k_off + ch), d = *reinterpret_cast<const float4*>(row + k_off + ch + 4);
        o.q[0] = a.x; o.q[1] = a.y; o.q[2] = a.z; o.q[3] = a.w; o.q[4] = b.x; o.q[5] = b.y; o.q[6] = b.z; o.q[7] = b.w;
        o.k[0] = c.x; o.k[1] = c.y; o.k[2] = c.z; o.k[3] = c.w; o.k[4] = d.x; o.k[5] = d.y; o.k[6] = d.z; o.k[7] = d.w;
    } else {
#pragma unroll
        for (int i = 0; i < DKPT; ++i) {
            const bool in = ch + i < dk;
            o.q[i] = in ? row[q_off + ch + i] : 0.f;
            o.k[i] = in ? row[k_off + ch + i] : 0.f;
        }
    }
    o.v = row[v_off];
    if (raw) {
#pragma unroll
        for (int i = 0; i < DKPT; ++i) {
            o.q[i] = silu_f(o.q[i]);
            o.k[i] = silu_f(o.k[i]);
        }
        o.v = silu_f(o.v);
    }
}

// Long portions go in runs of RUN tokens (the host's choice: shorter runs for shorter portions, so that the launches
// still fill the chip), all runs at once, in three launches:
//   1. every run on its own from an empty memory (LOCAL): its tokens' read-outs of the run's own keys, and what the run
//      adds to the memory, L_r = sum_s decay^(last - s) k_s v_s^T, into `runs` [run][H][dv][dkp];
//   2. decay_chain_kernel walks the runs of a sequence in order, element by element: the memory at the start of run r
//      takes L_r's place, S <- decay^len S + L_r goes on, and the state slot gets the end;
//   3. decay_carry_kernel adds what the memory at a run's start gives its tokens: o_t += decay^(i + 1) S_start^T q_t.
// Run r of sequence b lies at index q_start[b] / RUN + b + r: at most T / RUN + B runs in a step.

template <bool LOCAL>
__global__ void __launch_bounds__(256)
decay_attention_kernel(const float* __restrict__ act, int act_stride, const float* __restrict__ decay, float* __restrict__ state,
                       size_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                       const int32_t* __restrict__ state_slot, float* __restrict__ out, int H, int dk, int dv, int parts,
                       float* __restrict__ runs, int xblocks, bool raw, int RUN) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int cols = WAVE / parts;
    const int part = lane % parts;
    const int run = LOCAL ? blockIdx.x / xblocks : 0, xb = LOCAL ? blockIdx.x % xblocks : blockIdx.x;
    const int c = (xb * (blockDim.x / WAVE) + wave) * cols + lane / parts;
    const int first = run * RUN;                  // place in the portion of this block's first token
    const int n = LOCAL ? min(q_len[b] - first, RUN) : q_len[b];
    if (c >= dv || n <= 0) return;               // whole groups of `parts` lanes leave together
    const int dkp = parts * DKPT, ch = part * DKPT;
    float* srow = LOCAL ? runs + (static_cast<size_t>(q_start[b] / RUN + b + run) * H * dv + static_cast<size_t>(h) * dv + c) * dkp + ch
                        : state + static_cast<size_t>(state_slot[b]) * state_stride + (static_cast<size_t>(h) * dv + c) * dkp + ch;
    float S[DKPT];
    if (LOCAL) {
#pragma unroll
        for (int i = 0; i < DKPT; ++i) S[i] = 0.f;
    } else {
        const float4 a = *reinterpret_cast<const float4*>(srow), d = *reinterpret_cast<const float4*>(srow + 4);
        S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = d.x; S[5] = d.y; S[6] = d.z; S[7] = d.w;
    }
    const float w = decay[h];
    const int q_off = h * dk, k_off = H * dk + h * dk, v_off = 2 * H * dk + h * dv + c;
    const bool whole = dk % DKPT == 0 && ch + DKPT <= dk && act_stride % 4 == 0;
    const bool idle = ch >= dk;                   // a lane that holds padding only
    const int t0 = q_start[b] + first;
    DecayOperands cur, nxt;
    if (!idle) decay_load(cur, act + static_cast<size_t>(t0) * act_stride, q_off, k_off, v_off, ch, dk, whole, raw);
    for (int r = 0; r < n; ++r) {
        if (!idle && r + 1 < n) decay_load(nxt, act + static_cast<size_t>(t0 + r + 1) * act_stride, q_off, k_off, v_off, ch, dk, whole, raw);
        float sum = 0.f;
        if (!idle) {
#pragma unroll
            for (int i = 0; i < DKPT; ++i) {
                S[i] = w * S[i] + cur.k[i] * cur.v;
                sum += S[i] * cur.q[i];
            }
        }
        sum = parts_sum(sum, parts);
        if (part == 0) out[static_cast<size_t>(t0 + r) * (H * dv) + h * dv + c] = sum;
        cur = nxt;
    }
    // (a lane of padding writes back the zeros it holds: the chain over the runs reads every element)
    *reinterpret_cast<float4*>(srow) = make_float4(S[0], S[1], S[2], S[3]);
    *reinterpret_cast<float4*>(srow + 4) = make_float4(S[4], S[5], S[6], S[7]);
}

// step 2 of the runs: one thread an element of the memory [H][dv][dkp]
__global__ void decay_chain_kernel(float* __restrict__ runs, const float* __restrict__ decay, float* __restrict__ state,
                                   size_t state_stride, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                   const int32_t* __restrict__ state_slot, int per_head, int elems, int RUN) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    const int n = q_len[b];
    if (e >= elems || n <= 0) return;
    const float w = decay[e / per_head];
    const float w_run = powf(w, static_cast<float>(RUN));
    float* at = runs + static_cast<size_t>(q_start[b] / RUN + b) * elems + e;
    float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride + e;
    float S = *srow;
    const int n_runs = (n + RUN - 1) / RUN;
    for (int r = 0; r < n_runs; ++r) {
        const float add = at[static_cast<size_t>(r) * elems];
        at[static_cast<size_t>(r) * elems] = S;
        const int len = min(RUN, n - r * RUN);
        S = (len == RUN ? w_run : powf(w, static_cast<float>(len))) * S + add;
    }
    *srow = S;
}

// step 3 of the runs: the same threads as step 1, each with its eight numbers of the memory at the run's start
__global__ void __launch_bounds__(256)
decay_carry_kernel(const float* __restrict__ act, int act_stride, const float* __restrict__ decay, const float* __restrict__ runs,
                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out, int H, int dk,
                   int dv, int parts, int xblocks, int RUN) {
    const int b = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int cols = WAVE / parts;
    const int part = lane % parts;
    const int run = blockIdx.x / xblocks, xb = blockIdx.x % xblocks;
    const int c = (xb * (blockDim.x / WAVE) + wave) * cols + lane / parts;
    const int first = run * RUN;
    const int n = min(q_len[b] - first, RUN);
    if (c >= dv || n <= 0) return;
    const int dkp = parts * DKPT, ch = part * DKPT;
    const float* srow = runs + (static_cast<size_t>(q_start[b] / RUN + b + run) * H * dv + static_cast<size_t>(h) * dv + c) * dkp + ch;
    float S[DKPT];
    {
        const float4 a = *reinterpret_cast<const float4*>(srow), d = *reinterpret_cast<const float4*>(srow + 4);
        S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = d.x; S[5] = d.y; S[6] = d.z; S[7] = d.w;
    }
    const float w = decay[h];
    const int q_off = h * dk + ch;
    const bool whole = dk % DKPT == 0 && ch + DKPT <= dk && act_stride % 4 == 0;
    const bool idle = ch >= dk;
    const int t0 = q_start[b] + first;
    float faded = 1.f;
    for (int r = 0; r < n; ++r) {
        const float* row = act + static_cast<size_t>(t0 + r) * act_stride + q_off;
        float sum = 0.f;
        if (!idle) {
            if (whole) {
                const float4 a = *reinterpret_cast<const float4*>(row), d = *reinterpret_cast<const float4*>(row + 4);
                sum = S[0] * a.x + S[1] * a.y + S[2] * a.z + S[3] * a.w + S[4] * d.x + S[5] * d.y + S[6] * d.z + S[7] * d.w;
            } else {
#pragma unroll
                for (int i = 0; i < DKPT; ++i) sum += ch + i < dk ? S[i] * row[i] : 0.f;
            }
        }
        sum = parts_sum(sum, parts);
        faded *= w;
        if (part == 0) out[static_cast<size_t>(t0 + r) * (H * dv) + h * dv + c] += faded * sum;
    }
}

NI_EXPORT int ni_decay_attention_parts(int dk) {
    int parts = 1;
    while (parts * DKPT < dk) parts *= 2;
    return parts <= WAVE ? parts : 0;
}

// `raw` 1 (token by token only): `act` holds the projections and silu is applied as they are read.
// `max_q_len` bounds the portions of the step; `runs` (float32, (T / RUN + B) * H * dv * dkp, or null) switches the
// runs on: without it every sequence is walked token by token from its state.
NI_EXPORT int ni_decay_attention(const void* act, int act_stride, const void* decay, void* state, size_t state_stride,
                                 const void* q_start, const void* q_len, const void* state_slot, void* out, int T, int B,
                                 int H, int dk, int dv, int max_q_len, void* runs, int RUN, int raw, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (raw && runs) return -1;                   // the runs read their operands twice: they take them with silu applied
    const int parts = ni_decay_attention_parts(dk);
    if (!parts || act_stride < 2 * H * dk + H * dv || state_stride < static_cast<size_t>(H) * dv * parts * DKPT) return -1;
    if (reinterpret_cast<uintptr_t>(state) % 16 || state_stride % 4 || reinterpret_cast<uintptr_t>(act) % 16) return -1;
    const int cols = 4 * (WAVE / parts);
    const int xblocks = (dv + cols - 1) / cols;
    if (!runs) {
        dim3 grid(xblocks, H, B);
        decay_attention_kernel<false><<<grid, 256, 0, stream>>>((const float*)act, act_stride, (const float*)decay, (float*)state,
            state_stride, (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot, (float*)out, H, dk, dv, parts,
            nullptr, xblocks, raw != 0, 0);
        return NI_LAUNCH_RESULT();
    }
    if (max_q_len < 1 || max_q_len > T || RUN < 1 || reinterpret_cast<uintptr_t>(runs) % 16) return -1;
    const int n_runs = (max_q_len + RUN - 1) / RUN;
    dim3 grid(xblocks * n_runs, H, B);
    decay_attention_kernel<true><<<grid, 256, 0, stream>>>((const float*)act, act_stride, (const float*)decay, (float*)state,
        state_stride, (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot, (float*)out, H, dk, dv, parts,
        (float*)runs, xblocks, false, RUN);
    const int elems = H * dv * parts * DKPT;
    dim3 chain(blocks_of(elems, 256), B);
    decay_chain_kernel<<<chain, 256, 0, stream>>>((float*)runs, (const float*)decay, (float*)state, state_stride, (const int32_t*)q_start,
                                                  (const int32_t*)q_len, (const int32_t*)state_slot, dv * parts * DKPT, elems, RUN);
    decay_carry_kernel<<<grid, 256, 0, stream>>>((const float*)act, act_stride, (const float*)decay, (const float*)runs,
                                                 (const int32_t*)q_start, (const int32_t*)q_len, (float*)out, H, dk, dv, parts, xblocks, RUN);
    return NI_LAUNCH_RESULT();
}

// y[t, :] = o[t, :] / sqrt(mean(o[t, :]^2) + eps) * w * sigmoid(gate[t, :]) * out_scale, in the type T.
// One workgroup a token; gate rows have a stride of their own (they are columns of a wider projection).
template <typename T>
__global__ void __launch_bounds__(256)
gated_rmsnorm_kernel(const float* __restrict__ o, const float* __restrict__ gate, int gate_stride, const float* __restrict__ w,
                     T* __restrict__ y, int n, float eps, float out_scale) {
    __shared__ float scratch[8];
    const int t = blockIdx.x;
    const float* row = o + static_cast<size_t>(t) * n;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss += row[i] * row[i];
    const float r = out_scale / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
    const float* g = gate + static_cast<size_t>(t) * gate_stride;
    // a token is taken by gridDim.y workgroups, each with its share of the elements (and the whole row's sum of squares)
    const int per = (n + gridDim.y - 1) / gridDim.y;
    for (int i = blockIdx.y * per + threadIdx.x; i < min(n, (blockIdx.y + 1) * per); i += blockDim.x)
        st(y + static_cast<size_t>(t) * n + i, row[i] * r * w[i] * sigmoid_f(g[i]));
}

NI_EXPORT int ni_gated_rmsnorm(const void* o, const void* gate, int gate_stride, const void* w, void* y, int T, int n, float eps,
                               float out_scale, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (gate_stride < n) return -1;
    // few tokens: a row's elements over several workgroups (one workgroup walking a long row alone is a chain of round trips)
    const dim3 grid(T, T >= 64 ? 1 : std::max(1, std::min(16, (n + 255) / 256)));
    if (dtype == 0)
        gated_rmsnorm_kernel<float><<<grid, 256, 0, stream>>>((const float*)o, (const float*)gate, gate_stride, (const float*)w, (float*)y, n, eps, out_scale);
    else
        gated_rmsnorm_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)o, (const float*)gate, gate_stride, (const float*)w, (bf16_t*)y, n, eps, out_scale);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- causal convolution per channel, then silu
//   u[t, c] = silu(bias[c] + sum_j w[c, j] * x[t - (taps - 1 - j), c])      the last tap is the token's own input
// x is the first `inner` columns of xz float32 [T, xz_stride].  Inputs before a portion's first row come from
// `tail` (per slot [(taps - 1)][inner], the oldest first; zero for a new sequence), which conv_tail_kernel moves on
// afterwards, in a launch of its own (a step of single tokens, `single`, moves it on in the first kernel).  u goes out as float32 (for the recurrence) and, if asked for, in the compute
// type (for the product that follows).
template <typename T>
__global__ void conv_silu_kernel(const float* __restrict__ xz, int xz_stride, const float* __restrict__ w, const float* __restrict__ bias,
                                 float* __restrict__ state, size_t state_stride, size_t tail_off,
                                 const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
                                 const int32_t* __restrict__ state_slot, float* __restrict__ u32, T* __restrict__ uc,
                                 int inner, int taps, size_t total, bool single) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int t = static_cast<int>(i / inner), c = static_cast<int>(i % inner);
    const int b = seq_of_token[t];
    const int r = t - q_start[b];                 // place of the token in its portion
    float* tail = state + static_cast<size_t>(state_slot[b]) * state_stride + tail_off;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int back = taps - 1 - j;            // how many tokens before this one
        const float x = r - back >= 0 ? xz[static_cast<size_t>(t - back) * xz_stride + c]
                                      : tail[static_cast<size_t>(taps - 1 + r - back) * inner + c];
        acc += w[static_cast<size_t>(c) * taps + j] * x;
    }
    const float v = silu_f(acc);
    u32[i] = v;
    if (uc) st(uc + i, v);
    if (single) {        // every sequence brings one token: this thread alone reads and writes its channel's column of the tail
        for (int j = 0; j + 2 < taps; ++j) tail[static_cast<size_t>(j) * inner + c] = tail[static_cast<size_t>(j + 1) * inner + c];
        if (taps > 1) tail[static_cast<size_t>(taps - 2) * inner + c] = xz[static_cast<size_t>(t) * xz_stride + c];
    }
}

// the last taps - 1 inputs of every sequence of the step, oldest first; a thread moves one channel's column
__global__ void conv_tail_kernel(const float* __restrict__ xz, int xz_stride, float* __restrict__ state, size_t state_stride,
                                 size_t tail_off, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                 const int32_t* __restrict__ state_slot, int inner, int taps, int B) {
    const int c = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    if (c >= inner || b >= B) return;
    const int n = q_len[b], keep = taps - 1;
    if (n <= 0) return;
    float* tail = state + static_cast<size_t>(state_slot[b]) * state_stride + tail_off;
    for (int j = 0; j < keep; ++j) {              // ascending: what is read lies at or above what has been written
        const int idx = n - keep + j;             // place in the portion of the input that ends up at j
        tail[static_cast<size_t>(j) * inner + c] = idx >= 0 ? xz[static_cast<size_t>(q_start[b] + idx) * xz_stride + c]
                                                            : tail[static_cast<size_t>(keep + idx) * inner + c];
    }
}

NI_EXPORT int ni_conv_silu(const void* xz, int xz_stride, const void* w, const void* bias, void* state, size_t state_stride,
                           size_t tail_off, const void* seq_of_token, const void* q_start, const void* q_len, const void* state_slot,
                           void* u32, void* uc, int T, int B, int inner, int taps, int single, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * inner;
    if (total == 0 || B <= 0) return 0;
    if (taps < 1 || xz_stride < inner || state_stride < tail_off + static_cast<size_t>(taps - 1) * inner) return -1;
    if (single && T != B) return -1;              // a step of single tokens has one row a sequence
    if (dtype == 0)
        conv_silu_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)xz, xz_stride, (const float*)w, (const float*)bias,
            (float*)state, state_stride, tail_off, (const int32_t*)seq_of_token, (const int32_t*)q_start, (const int32_t*)state_slot,
            (float*)u32, (float*)uc, inner, taps, total, single != 0);
    else
        conv_silu_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)xz, xz_stride, (const float*)w, (const float*)bias,
            (float*)state, state_stride, tail_off, (const int32_t*)seq_of_token, (const int32_t*)q_start, (const int32_t*)state_slot,
            (float*)u32, (bf16_t*)uc, inner, taps, total, single != 0);
    if (taps > 1 && !single) {
        dim3 grid(blocks_of(inner, 256), B);
        conv_tail_kernel<<<grid, 256, 0, stream>>>((const float*)xz, xz_stride, (float*)state, state_stride, tail_off,
                                                   (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot, inner, taps, B);
    }
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the selective scan
//   dt = softplus(dt_pre[t, c] + dt_bias[c])
//   S[c, n] <- exp(dt A[c, n]) S[c, n] + dt u[t, c] B[t, n];   y[t, c] = (sum_n S[c, n] C[t, n] + D[c] u[t, c]) * silu(z[t, c])
// A float32 [inner][np] (negative; the padding zero), bc float32 [T, bc_stride] with B at column 0 and C at column N,
// z a column block of a wider projection (stride z_stride).  The state of a slot is [inner][np], np = parts * 4 >= N.
// A channel is held by `parts` neighbouring lanes with four of its numbers each; y in the type T.
#define SNPT 4

struct ScanOperands {
    float dt_pre, u, z, B[SNPT], C[SNPT];
};

__device__ __forceinline__ void scan_load(ScanOperands& o, const float* __restrict__ dt_pre, const float* __restrict__ u,
                                          const float* __restrict__ z, int z_stride, const float* __restrict__ bc, int bc_stride,
                                          size_t t, int c, int inner, int n0, int N, bool whole) {
    o.dt_pre = dt_pre[t * inner + c];
    o.u = u[t * inner + c];
    o.z = z[t * z_stride + c];
    const float* row = bc + t * bc_stride;
    if (whole) {
        const float4 a = *reinterpret_cast<const float4*>(row + n0), b = *reinterpret_cast<const float4*>(row + N + n0);
        o.B[0] = a.x; o.B[1] = a.y; o.B[2] = a.z; o.B[3] = a.w;
        o.C[0] = b.x; o.C[1] = b.y; o.C[2] = b.z; o.C[3] = b.w;
    } else {
#pragma unroll
        for (int i = 0; i < SNPT; ++i) {
            const bool in = n0 + i < N;
            o.B[i] = in ? row[n0 + i] : 0.f;
            o.C[i] = in ? row[N + n0 + i] : 0.f;
        }
    }
}

// Long portions go in runs of RUN tokens, all runs at once, as the decay attention's do:
//   1. every run on its own from an empty state (LOCAL): sum_n S C of its own tokens' inputs into `y_local`, the step sizes
//      summed from the run's start into `dt_sum` (both float32 [T, inner]), the state the run ends with into `runs`;
//   2. scan_chain_kernel walks the runs of a sequence in order: the state at the start of run r takes the run's place,
//      S <- exp(A * dt_sum at the run's end) S + the run's own goes on, the state slot gets the end;
//   3. scan_carry_kernel adds what the state at a run's start gives its tokens, sum_n C[t, n] exp(A[c, n] dt_sum[t, c]) S_start[c, n],
//      then D u and the gate.
template <typename T, bool LOCAL>
__global__ void __launch_bounds__(256)
selective_scan_kernel(const float* __restrict__ dt_pre, const float* __restrict__ dt_bias, const float* __restrict__ u,
                      const float* __restrict__ z, int z_stride, const float* __restrict__ bc, int bc_stride,
                      const float* __restrict__ A, const float* __restrict__ D, float* __restrict__ state, size_t state_stride,
                      const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot,
                      T* __restrict__ y, int inner, int N, int parts, float* __restrict__ runs, float* __restrict__ y_local,
                      float* __restrict__ dt_sum, int xblocks, int RUN) {
    const int b = blockIdx.y;
    const int part = threadIdx.x % parts;
    const int run = LOCAL ? blockIdx.x / xblocks : 0, xb = LOCAL ? blockIdx.x % xblocks : blockIdx.x;
    const int c = (xb * blockDim.x + threadIdx.x) / parts;
    const int first = run * RUN;
    const int n = LOCAL ? min(q_len[b] - first, RUN) : q_len[b];
    if (c >= inner || n <= 0) return;            // whole groups of `parts` lanes leave together
    const int np = parts * SNPT, n0 = part * SNPT;
    float* srow = LOCAL ? runs + (static_cast<size_t>(q_start[b] / RUN + b + run) * inner + c) * np + n0
                        : state + static_cast<size_t>(state_slot[b]) * state_stride + static_cast<size_t>(c) * np + n0;
    float S[SNPT] = {0.f, 0.f, 0.f, 0.f};
    if (!LOCAL) {
        const float4 s4 = *reinterpret_cast<const float4*>(srow);
        S[0] = s4.x; S[1] = s4.y; S[2] = s4.z; S[3] = s4.w;
    }
    const float4 a4 = *reinterpret_cast<const float4*>(A + static_cast<size_t>(c) * np + n0);
    const float Ac[SNPT] = {a4.x, a4.y, a4.z, a4.w};
    const float bias = dt_bias[c], Dc = D[c];
    const bool whole = N % SNPT == 0 && n0 + SNPT <= N && bc_stride % 4 == 0;
    const size_t t0 = static_cast<size_t>(q_start[b] + first);
    float total = 0.f;
    ScanOperands cur, nxt;
    scan_load(cur, dt_pre, u, z, z_stride, bc, bc_stride, t0, c, inner, n0, N, whole);
    for (int r = 0; r < n; ++r) {
        if (r + 1 < n) scan_load(nxt, dt_pre, u, z, z_stride, bc, bc_stride, t0 + r + 1, c, inner, n0, N, whole);
        const float dt = softplus_f(cur.dt_pre + bias);
        const float du = dt * cur.u;
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < SNPT; ++i) {
            S[i] = expf(dt * Ac[i]) * S[i] + du * cur.B[i];
            sum += S[i] * cur.C[i];
        }
        sum = parts_sum(sum, parts);
        if (LOCAL) {
            total += dt;
            if (part == 0) {
                y_local[(t0 + r) * inner + c] = sum;
                dt_sum[(t0 + r) * inner + c] = total;
            }
        } else if (part == 0) {
            st(y + (t0 + r) * inner + c, (sum + Dc * cur.u) * silu_f(cur.z));
        }
        cur = nxt;
    }
    *reinterpret_cast<float4*>(srow) = make_float4(S[0], S[1], S[2], S[3]);
}

// step 2 of the runs: one thread an element of the state [inner][np]
__global__ void scan_chain_kernel(float* __restrict__ runs, const float* __restrict__ A, const float* __restrict__ dt_sum,
                                  float* __restrict__ state, size_t state_stride, const int32_t* __restrict__ q_start,
                                  const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot, int inner, int np, int RUN) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    const int n = q_len[b], elems = inner * np;
    if (e >= elems || n <= 0) return;
    const int c = e / np;
    const float a = A[e];
    float* at = runs + static_cast<size_t>(q_start[b] / RUN + b) * elems + e;
    float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride + e;
    float S = *srow;
    const int n_runs = (n + RUN - 1) / RUN;
    for (int r = 0; r < n_runs; ++r) {
        const float add = at[static_cast<size_t>(r) * elems];
        at[static_cast<size_t>(r) * elems] = S;
        const int last = min(n, (r + 1) * RUN) - 1;
        S = expf(a * dt_sum[static_cast<size_t>(q_start[b] + last) * inner + c]) * S + add;
    }
    *srow = S;
}

// step 3 of the runs: the same threads as step 1
template <typename T>
__global__ void __launch_bounds__(256)
scan_carry_kernel(const float* __restrict__ u, const float* __restrict__ z, int z_stride, const float* __restrict__ bc, int bc_stride,
                  const float* __restrict__ A, const float* __restrict__ D, const float* __restrict__ runs,
                  const float* __restrict__ y_local, const float* __restrict__ dt_sum, const int32_t* __restrict__ q_start,
                  const int32_t* __restrict__ q_len, T* __restrict__ y, int inner, int N, int parts, int xblocks, int RUN) {
    const int b = blockIdx.y;
    const int part = threadIdx.x % parts;
    const int run = blockIdx.x / xblocks, xb = blockIdx.x % xblocks;
    const int c = (xb * blockDim.x + threadIdx.x) / parts;
    const int first = run * RUN;
    const int n = min(q_len[b] - first, RUN);
    if (c >= inner || n <= 0) return;
    const int np = parts * SNPT, n0 = part * SNPT;
    const float4 s4 = *reinterpret_cast<const float4*>(runs + (static_cast<size_t>(q_start[b] / RUN + b + run) * inner + c) * np + n0);
    const float S[SNPT] = {s4.x, s4.y, s4.z, s4.w};
    const float4 a4 = *reinterpret_cast<const float4*>(A + static_cast<size_t>(c) * np + n0);
    const float Ac[SNPT] = {a4.x, a4.y, a4.z, a4.w};
    const float Dc = D[c];
    const bool whole = N % SNPT == 0 && n0 + SNPT <= N && bc_stride % 4 == 0;
    const size_t t0 = static_cast<size_t>(q_start[b] + first);
    for (int r = 0; r < n; ++r) {
        const size_t t = t0 + r;
        const float* row = bc + t * bc_stride + N + n0;
        float C[SNPT];
        if (whole) {
            const float4 c4 = *reinterpret_cast<const float4*>(row);
            C[0] = c4.x; C[1] = c4.y; C[2] = c4.z; C[3] = c4.w;
        } else {
#pragma unroll
            for (int i = 0; i < SNPT; ++i) C[i] = n0 + i < N ? row[i] : 0.f;
        }
        const float dts = dt_sum[t * inner + c];
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < SNPT; ++i) sum += C[i] * expf(Ac[i] * dts) * S[i];
        sum = parts_sum(sum, parts);
        if (part == 0) {
            const float uc = u[t * inner + c];
            st(y + t * inner + c, (y_local[t * inner + c] + sum + Dc * uc) * silu_f(z[t * z_stride + c]));
        }
    }
}

NI_EXPORT int ni_selective_scan_parts(int N) {
    int parts = 1;
    while (parts * SNPT < N) parts *= 2;
    return parts <= WAVE ? parts : 0;
}

template <typename T>
static void launch_scan(const void* dt_pre, const void* dt_bias, const void* u, const void* z, int z_stride, const void* bc, int bc_stride,
                        const void* A, const void* D, void* state, size_t state_stride, const void* q_start, const void* q_len,
                        const void* state_slot, void* y, int B, int inner, int N, int parts, int max_q_len, void* runs, void* y_local,
                        void* dt_sum, int RUN, hipStream_t stream) {
    const int xblocks = blocks_of(static_cast<size_t>(inner) * parts, 256);
    if (!runs) {
        dim3 grid(xblocks, B);
        selective_scan_kernel<T, false><<<grid, 256, 0, stream>>>((const float*)dt_pre, (const float*)dt_bias, (const float*)u, (const float*)z,
            z_stride, (const float*)bc, bc_stride, (const float*)A, (const float*)D, (float*)state, state_stride, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, (T*)y, inner, N, parts, nullptr, nullptr, nullptr, xblocks, 0);
        return;
    }
    const int n_runs = (max_q_len + RUN - 1) / RUN;
    dim3 grid(xblocks * n_runs, B);
    selective_scan_kernel<T, true><<<grid, 256, 0, stream>>>((const float*)dt_pre, (const float*)dt_bias, (const float*)u, (const float*)z,
        z_stride, (const float*)bc, bc_stride, (const float*)A, (const float*)D, (float*)state, state_stride, (const int32_t*)q_start,
        (const int32_t*)q_len, (const int32_t*)state_slot, (T*)y, inner, N, parts, (float*)runs, (float*)y_local, (float*)dt_sum, xblocks, RUN);
    dim3 chain(blocks_of(static_cast<size_t>(inner) * parts * SNPT, 256), B);
    scan_chain_kernel<<<chain, 256, 0, stream>>>((float*)runs, (const float*)A, (const float*)dt_sum, (float*)state, state_stride,
                                                 (const int32_t*)q_start, (const int32_t*)q_len, (const int32_t*)state_slot, inner, parts * SNPT, RUN);
    scan_carry_kernel<T><<<grid, 256, 0, stream>>>((const float*)u, (const float*)z, z_stride, (const float*)bc, bc_stride, (const float*)A,
        (const float*)D, (const float*)runs, (const float*)y_local, (const float*)dt_sum, (const int32_t*)q_start, (const int32_t*)q_len,
        (T*)y, inner, N, parts, xblocks, RUN);
}

// `runs` (float32, (T / RUN + B) * inner * np, or null) switches the runs on, with `y_local` and `dt_sum` (float32 [T, inner]
// each) and `max_q_len`, a bound on the portions of the step; without it every sequence is walked token by token from its state.
NI_EXPORT int ni_selective_scan(const void* dt_pre, const void* dt_bias, const void* u, const void* z, int z_stride, const void* bc,
                                int bc_stride, const void* A, const void* D, void* state, size_t state_stride, const void* q_start,
                                const void* q_len, const void* state_slot, void* y, int T, int B, int inner, int N, int max_q_len,
                                void* runs, void* y_local, void* dt_sum, int RUN, int dtype, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    const int parts = ni_selective_scan_parts(N);
    if (!parts || z_stride < inner || bc_stride < 2 * N || state_stride < static_cast<size_t>(inner) * parts * SNPT) return -1;
    if (reinterpret_cast<uintptr_t>(state) % 16 || state_stride % 4 || reinterpret_cast<uintptr_t>(A) % 16 ||
        reinterpret_cast<uintptr_t>(bc) % 16) return -1;
    if (runs && (!y_local || !dt_sum || max_q_len < 1 || max_q_len > T || RUN < 1 || reinterpret_cast<uintptr_t>(runs) % 16)) return -1;
    if (dtype == 0)
        launch_scan<float>(dt_pre, dt_bias, u, z, z_stride, bc, bc_stride, A, D, state, state_stride, q_start, q_len, state_slot, y, B,
                           inner, N, parts, max_q_len, runs, y_local, dt_sum, RUN, stream);
    else
        launch_scan<bf16_t>(dt_pre, dt_bias, u, z, z_stride, bc, bc_stride, A, D, state, state_stride, q_start, q_len, state_slot, y, B,
                            inner, N, parts, max_q_len, runs, y_local, dt_sum, RUN, stream);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- matrix memory with exponential gates
// Per head, with a memory S [dk, dv], a normaliser n [dk] and a running maximum m of the gates' logarithms, all float32:
//   li = cap tanh((zi + bi) / cap),  lf = logsigmoid(cap tanh((zf + bf) / cap))
//   m' = max(lf + m, li);  S <- exp(lf + m - m') S + exp(li - m') k v^T;  n likewise with k alone;  m <- m'
//   o = S^T q / (max(|n . q|, exp(-m)) + 1e-6)
// The normaliser is kept as one more value channel whose value is always 1: a slot's state is [H][dv + 1][dkp]
// (a column of key channels lies together, dkp = parts * 8 >= dk, padding zero) and then m [H].  proj float32
// [T, stride] holds q, k [H dk each], v [H dv] and the gates' pre-activations zi [H], zf [H] at given columns.  The
// recurrence kernels leave the raw read-outs [T, H (dv + 1)] (the last of a head is n . q) and m [T, H];
// memory_norm_kernel divides, norms every head, gates, and keeps the last m of every sequence in the state.
struct MemoryOperands {
    float q[DKPT], k[DKPT], v;
};

__device__ __forceinline__ float log_sigmoid_f(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__device__ __forceinline__ void memory_load(MemoryOperands& o, const float* __restrict__ row, int q_off, int k_off, int v_off,
                                            float q_scale, int ch, int dk, bool whole, bool ones) {
    if (whole) {
        const float4 a = *reinterpret_cast<const float4*>(row + q_off + ch), b = *reinterpret_cast<const float4*>(row + q_off + ch + 4);
        const float4 c = *reinterpret_cast<const float4*>(row + k_off + ch), d = *reinterpret_cast<const float4*>(row + k_off + ch + 4);
        o.q[0] = a.x; o.q[1] = a.y; o.q[2] = a.z; o.q[3] = a.w; o.q[4] = b.x; o.q[5] = b.y; o.q[6] = b.z; o.q[7] = b.w;
        o.k[0] = c.x; o.k[1] = c.y; o.k[2] = c.z; o.k[3] = c.w; o.k[4] = d.x; o.k[5] = d.y; o.k[6] = d.z; o.k[7] = d.w;
    } else {
#pragma unroll
        for (int i = 0; i < DKPT; ++i) {
            const bool in = ch + i < dk;
            o.q[i] = in ? row[q_off + ch + i] : 0.f;
            o.k[i] = in ? row[k_off + ch + i] : 0.f;
        }
    }
#pragma unroll
    for (int i = 0; i < DKPT; ++i) o.q[i] *= q_scale;
    o.v = ones ? 1.f : row[v_off];
}

// tokens whose gates a workgroup works out together, one a thread
constexpr int GATE_TOKENS = 256;

// Token by token from the state (LOCAL false), or a run of RUN tokens from an empty memory whose maximum starts at
// minus infinity (LOCAL true; the runs' layout is decay_attention_kernel's).  A LOCAL run also leaves, per token, the
// sum of lf since the run's start (`since`), and per run and head (its maximum at the end, that sum at the end).
template <bool LOCAL>
__global__ void __launch_bounds__(256)
memory_steps_kernel(const float* __restrict__ proj, int stride, int q_col, int k_col, int v_col, int z_col,
                    const float* __restrict__ gate_bias, float cap, float q_scale, const float* __restrict__ state,
                    float* __restrict__ state_out, size_t state_stride, const int32_t* __restrict__ q_start,
                    const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot, float* __restrict__ out,
                    float* __restrict__ m_out, float* __restrict__ since, float* __restrict__ run_ends, int H, int dk, int dv,
                    int parts, float* __restrict__ runs, int xblocks, int RUN) {
    // the gates are the same for every column of a head: the workgroup works them out once, GATE_TOKENS tokens at a
    // time and one a thread (li, lf), one thread walks the maxima (additions and comparisons only), and every thread
    // again makes its token's two factors exp(lf + m - m') and exp(li - m'), which the columns' lanes then read
    __shared__ float g_take[GATE_TOKENS], g_keep[GATE_TOKENS], g_m[GATE_TOKENS], g_passed[GATE_TOKENS];
    const int b = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int cols = WAVE / parts;
    const int part = lane % parts;
    const int run = LOCAL ? blockIdx.x / xblocks : 0, xb = LOCAL ? blockIdx.x % xblocks : blockIdx.x;
    const int c = (xb * (blockDim.x / WAVE) + wave) * cols + lane / parts;
    const int first = run * RUN;
    const int n = LOCAL ? min(q_len[b] - first, RUN) : q_len[b];
    const int dvn = dv + 1;
    if (n <= 0) return;                           // the whole workgroup
    const bool active = c < dvn;                  // a group of `parts` lanes holds a column or none
    const int dkp = parts * DKPT, ch = part * DKPT;
    const size_t heads_floats = static_cast<size_t>(H) * dvn * dkp;
    const size_t run_index = LOCAL ? static_cast<size_t>(q_start[b] / RUN + b + run) : 0;
    const size_t at = (static_cast<size_t>(h) * dvn + c) * dkp + ch;
    float S[DKPT];
#pragma unroll
    for (int i = 0; i < DKPT; ++i) S[i] = 0.f;
    float m = -INFINITY;
    if (!LOCAL) {
        const float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride;
        if (active) {
            const float4 a = *reinterpret_cast<const float4*>(srow + at), d = *reinterpret_cast<const float4*>(srow + at + 4);
            S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = d.x; S[5] = d.y; S[6] = d.z; S[7] = d.w;
        }
        m = srow[heads_floats + h];
    }
    const float bi = gate_bias[h], bf = gate_bias[H + h];
    const int q_off = q_col + h * dk, k_off = k_col + h * dk, v_off = v_col + h * dv + c, zi_off = z_col + h, zf_off = z_col + H + h;
    const bool whole = dk % DKPT == 0 && ch + DKPT <= dk && stride % 4 == 0 && q_col % 4 == 0 && k_col % 4 == 0;
    const bool idle = ch >= dk;                   // a lane that holds padding only
    const bool ones = c == dv;                    // the normaliser's column
    const bool scribe = xb == 0;                  // the one workgroup of (sequence, head, run) that writes the scalars
    const int t0 = q_start[b] + first;
    float passed = 0.f;                           // sum of lf since the run's start
    MemoryOperands cur, nxt;
    if (active) memory_load(cur, proj + static_cast<size_t>(t0) * stride, q_off, k_off, v_off, q_scale, ch, dk, whole && !idle, ones);
    for (int base = 0; base < n; base += GATE_TOKENS) {
        const int cn = min(n - base, GATE_TOKENS);
        const int r_own = threadIdx.x;
        if (r_own < cn) {
            const float* row = proj + static_cast<size_t>(t0 + base + r_own) * stride;
            g_take[r_own] = cap * tanhf((row[zi_off] + bi) / cap);                     // li
            g_keep[r_own] = log_sigmoid_f(cap * tanhf((row[zf_off] + bf) / cap));      // lf
        }
        __syncthreads();
        if (threadIdx.x == 0) {
            float mm = m, pp = passed;
            for (int r = 0; r < cn; ++r) {
                mm = fmaxf(g_keep[r] + mm, g_take[r]);
                pp += g_keep[r];
                g_m[r] = mm;
                g_passed[r] = pp;
            }
        }
        __syncthreads();
        if (r_own < cn) {
            const float before = r_own ? g_m[r_own - 1] : m, now = g_m[r_own];
            const float li = g_take[r_own], lf = g_keep[r_own];
            g_keep[r_own] = expf(lf + before - now);
            g_take[r_own] = expf(li - now);
            if (scribe) {
                m_out[static_cast<size_t>(t0 + base + r_own) * H + h] = now;
                if (LOCAL) since[static_cast<size_t>(t0 + base + r_own) * H + h] = g_passed[r_own];
            }
        }
        __syncthreads();
        if (active) {
            for (int r = 0; r < cn; ++r) {
                if (base + r + 1 < n)
                    memory_load(nxt, proj + static_cast<size_t>(t0 + base + r + 1) * stride, q_off, k_off, v_off, q_scale, ch, dk,
                                whole && !idle, ones);
                const float keep = g_keep[r], take = g_take[r] * cur.v;
                float sum = 0.f;
                if (!idle) {
#pragma unroll
                    for (int i = 0; i < DKPT; ++i) {
                        S[i] = keep * S[i] + take * cur.k[i];
                        sum += S[i] * cur.q[i];
                    }
                }
                sum = parts_sum(sum, parts);
                if (part == 0) out[static_cast<size_t>(t0 + base + r) * (H * dvn) + h * dvn + c] = sum;
                cur = nxt;
            }
        }
        m = g_m[cn - 1];
        passed = g_passed[cn - 1];
        __syncthreads();                          // the next tokens' gates take these places
    }
    if (active) {
        float* dst = LOCAL ? runs + run_index * heads_floats + at : state_out + static_cast<size_t>(state_slot[b]) * state_stride + at;
        *reinterpret_cast<float4*>(dst) = make_float4(S[0], S[1], S[2], S[3]);
        *reinterpret_cast<float4*>(dst + 4) = make_float4(S[4], S[5], S[6], S[7]);
    }
    if (LOCAL && scribe && threadIdx.x == 0) {
        run_ends[(run_index * H + h) * 2] = m;
        run_ends[(run_index * H + h) * 2 + 1] = passed;
    }
}

// step 2 of the runs: one thread an element of [H][dv + 1][dkp]; the memory at the start of run r takes the place of
// what the run adds, and run_starts gets the maximum at the start of every run
__global__ void memory_chain_kernel(float* __restrict__ runs, const float* __restrict__ run_ends, float* __restrict__ run_starts,
                                    float* __restrict__ state, size_t state_stride, const int32_t* __restrict__ q_start,
                                    const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot, int per_head, int H,
                                    int elems, int RUN) {
    const int e = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
    const int n = q_len[b];
    if (e >= elems || n <= 0) return;
    const int h = e / per_head;
    const size_t base = static_cast<size_t>(q_start[b] / RUN + b);
    float* srow = state + static_cast<size_t>(state_slot[b]) * state_stride;
    float S = srow[e];
    float m = srow[elems + h];
    const int n_runs = (n + RUN - 1) / RUN;
    for (int r = 0; r < n_runs; ++r) {
        float* at = runs + (base + r) * elems + e;
        const float add = *at;
        *at = S;
        if (e % per_head == 0) run_starts[(base + r) * H + h] = m;
        const float end_max = run_ends[((base + r) * H + h) * 2], passed = run_ends[((base + r) * H + h) * 2 + 1];
        const float m_new = fmaxf(passed + m, end_max);
        S = expf(passed + m - m_new) * S + expf(end_max - m_new) * add;
        m = m_new;
    }
    srow[e] = S;          // (the maximum itself is kept by memory_norm_kernel: other threads of this launch still read it)
}

// step 3 of the runs: what the memory at a run's start gives its tokens, and every token's own maximum
__global__ void __launch_bounds__(256)
memory_carry_kernel(const float* __restrict__ proj, int stride, int q_col, float q_scale, const float* __restrict__ runs,
                    const float* __restrict__ run_starts, const float* __restrict__ local_max, const float* __restrict__ since,
                    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, float* __restrict__ out,
                    float* __restrict__ m_out, int H, int dk, int dv, int parts, int xblocks, int RUN) {
    // what a token's own read-out and what the memory at the run's start weigh, once a workgroup and token
    __shared__ float f_own[GATE_TOKENS], f_before[GATE_TOKENS];
    const int b = blockIdx.z, h = blockIdx.y;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    const int cols = WAVE / parts;
    const int part = lane % parts;
    const int run = blockIdx.x / xblocks, xb = blockIdx.x % xblocks;
    const int c = (xb * (blockDim.x / WAVE) + wave) * cols + lane / parts;
    const int first = run * RUN;
    const int n = min(q_len[b] - first, RUN);
    const int dvn = dv + 1;
    if (n <= 0) return;                           // the whole workgroup
    const bool active = c < dvn;
    const int dkp = parts * DKPT, ch = part * DKPT;
    const size_t run_index = static_cast<size_t>(q_start[b] / RUN + b + run);
    const float* srow = runs + run_index * H * dvn * dkp + (static_cast<size_t>(h) * dvn + c) * dkp + ch;
    float S[DKPT];
#pragma unroll
    for (int i = 0; i < DKPT; ++i) S[i] = 0.f;
    if (active) {
        const float4 a = *reinterpret_cast<const float4*>(srow), d = *reinterpret_cast<const float4*>(srow + 4);
        S[0] = a.x; S[1] = a.y; S[2] = a.z; S[3] = a.w; S[4] = d.x; S[5] = d.y; S[6] = d.z; S[7] = d.w;
    }
    const float m0 = run_starts[run_index * H + h];
    const int q_off = q_col + h * dk + ch;
    const bool whole = dk % DKPT == 0 && ch + DKPT <= dk && stride % 4 == 0 && q_col % 4 == 0;
    const bool idle = ch >= dk;
    const bool scribe = xb == 0;
    const int t0 = q_start[b] + first;
    for (int base = 0; base < n; base += GATE_TOKENS) {
        const int cn = min(n - base, GATE_TOKENS);
        if (threadIdx.x < cn) {
            const size_t th = static_cast<size_t>(t0 + base + threadIdx.x) * H + h;
            const float own = local_max[th], before = since[th] + m0;
            const float m = fmaxf(before, own);
            f_own[threadIdx.x] = expf(own - m);
            f_before[threadIdx.x] = expf(before - m);
            if (scribe) m_out[th] = m;
        }
        __syncthreads();
        if (active) {
            for (int r = 0; r < cn; ++r) {
                const float* row = proj + static_cast<size_t>(t0 + base + r) * stride + q_off;
                float sum = 0.f;
                if (!idle) {
                    if (whole) {
                        const float4 a = *reinterpret_cast<const float4*>(row), d = *reinterpret_cast<const float4*>(row + 4);
                        sum = S[0] * a.x + S[1] * a.y + S[2] * a.z + S[3] * a.w + S[4] * d.x + S[5] * d.y + S[6] * d.z + S[7] * d.w;
                    } else {
#pragma unroll
                        for (int i = 0; i < DKPT; ++i) sum += ch + i < dk ? S[i] * row[i] : 0.f;
                    }
                }
                sum = parts_sum(sum, parts) * q_scale;
                if (part == 0) {
                    float* o = out + static_cast<size_t>(t0 + base + r) * (H * dvn) + h * dvn + c;
                    *o = f_own[r] * *o + f_before[r] * sum;
                }
            }
        }
        __syncthreads();                          // the next tokens' factors take these places
    }
}

// y[t, h dv + c] = N_h(o / (max(|n . q|, exp(-m)) + 1e-6)) * w * sigmoid(gate): N_h divides a head's dv numbers by their
// root mean square.  raw float32 [T, H (dv + 1)], m float32 [T, H]; a token is taken by gridDim.y workgroups, a wavefront a
// head at a time (a step of few tokens gives every head a wavefront of its own: one workgroup walking sixteen heads,
// four at a time with dependent reads, took 11.7 us a decode step).  The last token of every sequence's portion leaves its m in the state (behind the memories, at `m_off`).
template <typename T>
__global__ void __launch_bounds__(256)
memory_norm_kernel(const float* __restrict__ raw, const float* __restrict__ m_of, const float* __restrict__ gate, int gate_stride,
                   const float* __restrict__ w, T* __restrict__ y, float* __restrict__ state, size_t state_stride, size_t m_off,
                   const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                   const int32_t* __restrict__ state_slot, int H, int dv, float eps) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
    const int dvn = dv + 1;
    const int b = seq_of_token[t];
    const bool last = t == q_start[b] + q_len[b] - 1;
    for (int h = blockIdx.y * waves + wave; h < H; h += waves * gridDim.y) {
        const float* row = raw + static_cast<size_t>(t) * H * dvn + static_cast<size_t>(h) * dvn;
        const float m = m_of[static_cast<size_t>(t) * H + h];
        const float inv = 1.0f / (fmaxf(fabsf(row[dv]), expf(-m)) + 1e-6f);
        float ss = 0.f;
        for (int c = lane; c < dv; c += WAVE) {
            const float v = row[c] * inv;
            ss += v * v;
        }
        const float r = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(dv) + eps);
        const float* g = gate + static_cast<size_t>(t) * gate_stride + h * dv;
        for (int c = lane; c < dv; c += WAVE)
            st(y + static_cast<size_t>(t) * H * dv + h * dv + c, (row[c] * inv) * r * w[h * dv + c] * sigmoid_f(g[c]));
        if (last && lane == 0) state[static_cast<size_t>(state_slot[b]) * state_stride + m_off + h] = m;
    }
}

NI_EXPORT int ni_memory_norm(const void* raw, const void* m_of, const void* gate, int gate_stride, const void* w, void* y,
                             void* state, size_t state_stride, size_t m_off, const void* seq_of_token, const void* q_start,
                             const void* q_len, const void* state_slot, int T, int H, int dv, float eps, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (gate_stride < H * dv || state_stride < m_off + H) return -1;
    const int threads = H >= 4 ? 256 : 64 * H;
    const dim3 grid(T, T >= 64 ? 1 : std::min(16, (H * 64 + threads - 1) / threads));
    if (dtype == 0)
        memory_norm_kernel<float><<<grid, threads, 0, stream>>>((const float*)raw, (const float*)m_of, (const float*)gate, gate_stride,
            (const float*)w, (float*)y, (float*)state, state_stride, m_off, (const int32_t*)seq_of_token, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, H, dv, eps);
    else
        memory_norm_kernel<bf16_t><<<grid, threads, 0, stream>>>((const float*)raw, (const float*)m_of, (const float*)gate, gate_stride,
            (const float*)w, (bf16_t*)y, (float*)state, state_stride, m_off, (const int32_t*)seq_of_token, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, H, dv, eps);
    return NI_LAUNCH_RESULT();
}

// `scalars` (float32, 3 T H + 3 (T / RUN + B) H; the first T H only without runs): the tokens' local maxima and sums of
// lf, and the runs' ends and starts.  `runs` (float32, (T / RUN + B) H (dv + 1) dkp, or null) switches the runs on.
// m_out float32 [T, H]; out float32 [T, H (dv + 1)].
NI_EXPORT int ni_gated_memory(const void* proj, int stride, int q_col, int k_col, int v_col, int z_col, const void* gate_bias,
                              float cap, float q_scale, void* state, size_t state_stride, const void* q_start, const void* q_len,
                              const void* state_slot, void* out, void* m_out, int T, int B, int H, int dk, int dv, int max_q_len,
                              void* runs, void* scalars, int RUN, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    const int parts = ni_decay_attention_parts(dk);
    const int dvn = dv + 1;
    const size_t heads_floats = static_cast<size_t>(H) * dvn * parts * DKPT;
    if (!parts || state_stride < heads_floats + H || !(cap > 0.f)) return -1;
    if (stride < q_col + H * dk || stride < k_col + H * dk || stride < v_col + H * dv || stride < z_col + 2 * H) return -1;
    if (reinterpret_cast<uintptr_t>(state) % 16 || state_stride % 4 || reinterpret_cast<uintptr_t>(proj) % 16) return -1;
    const int cols = 4 * (WAVE / parts);
    const int xblocks = (dvn + cols - 1) / cols;
    if (!runs) {
        dim3 grid(xblocks, H, B);
        memory_steps_kernel<false><<<grid, 256, 0, stream>>>((const float*)proj, stride, q_col, k_col, v_col, z_col,
            (const float*)gate_bias, cap, q_scale, (const float*)state, (float*)state, state_stride, (const int32_t*)q_start,
            (const int32_t*)q_len, (const int32_t*)state_slot, (float*)out, (float*)m_out, nullptr, nullptr, H, dk, dv, parts, nullptr,
            xblocks, 0);
        return NI_LAUNCH_RESULT();
    }
    if (max_q_len < 1 || max_q_len > T || RUN < 1 || !scalars || reinterpret_cast<uintptr_t>(runs) % 16) return -1;
    const size_t max_runs = static_cast<size_t>(T / RUN + B);
    float* local_max = (float*)scalars;
    float* since = local_max + static_cast<size_t>(T) * H;
    float* run_ends = since + static_cast<size_t>(T) * H;
    float* run_starts = run_ends + max_runs * H * 2;
    const int n_runs = (max_q_len + RUN - 1) / RUN;
    dim3 grid(xblocks * n_runs, H, B);
    memory_steps_kernel<true><<<grid, 256, 0, stream>>>((const float*)proj, stride, q_col, k_col, v_col, z_col,
        (const float*)gate_bias, cap, q_scale, nullptr, nullptr, 0, (const int32_t*)q_start, (const int32_t*)q_len,
        (const int32_t*)state_slot, (float*)out, local_max, since, run_ends, H, dk, dv, parts, (float*)runs, xblocks, RUN);
    const int elems = static_cast<int>(heads_floats);
    dim3 chain(blocks_of(elems, 256), B);
    memory_chain_kernel<<<chain, 256, 0, stream>>>((float*)runs, run_ends, run_starts, (float*)state, state_stride, (const int32_t*)q_start,
                                                   (const int32_t*)q_len, (const int32_t*)state_slot, dvn * parts * DKPT, H, elems, RUN);
    memory_carry_kernel<<<grid, 256, 0, stream>>>((const float*)proj, stride, q_col, q_scale, (const float*)runs, run_starts, local_max,
                                                  since, (const int32_t*)q_start, (const int32_t*)q_len, (float*)out, (float*)m_out, H,
                                                  dk, dv, parts, xblocks, RUN);
    return NI_LAUNCH_RESULT();
}
