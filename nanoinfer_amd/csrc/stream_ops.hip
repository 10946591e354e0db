// Kernels around the residual stream and the routed feed-forward for gfx950: an embedding that
// scales its rows and adds a learned position row, sums onto the float32 stream, a token's side
// input, the router's choice, and the products of the chosen experts for steps of few rows.
//
// Conventions as in ops.hip: the stream is float32, what feeds a matrix product is the compute
// type (float or bfloat16), all arithmetic is float32, every entry point returns 0 or a hipError_t.
#include "common.h"

#include <algorithm>

static inline unsigned blocks_of(size_t n, unsigned per) { return static_cast<unsigned>((n + per - 1) / per); }
static inline bool aligned16(const void* a, const void* b) {
    return (reinterpret_cast<uintptr_t>(a) % 16 == 0) && (reinterpret_cast<uintptr_t>(b) % 16 == 0);
}

__device__ __forceinline__ float gelu_tanh_f(float z) {
    // 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
    const float c = 0.7978845608028654f;
    return 0.5f * z * (1.0f + tanhf(c * (z + 0.044715f * z * z * z)));
}

// ---------------------------------------------------------------- embedding: row * scale + position row
template <typename T>
__global__ void embed_scaled_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                    const T* __restrict__ table, const T* __restrict__ pos_table, float* __restrict__ out,
                                    int d, int vocab, int max_pos, float scale) {
    const int t = blockIdx.x;
    const int id = ids[t];
    if (id < 0 || id >= vocab) return;      // unreachable after the host's check
    const T* row = table + static_cast<size_t>(id) * d;
    float* o = out + static_cast<size_t>(t) * d;
    const T* prow = nullptr;
    if (pos_table) {
        const int p = positions[t];
        if (p < 0 || p >= max_pos) return;  // the runner refuses a request before it reaches the last position
        prow = pos_table + static_cast<size_t>(p) * d;
    }
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = ld(row + i) * scale;
        if (prow) v += ld(prow + i);
        o[i] = v;
    }
}

NI_EXPORT int ni_embed_scaled(const void* ids, const void* positions, const void* table, const void* pos_table, void* out,
                              int T, int d, int vocab, int max_pos, float scale, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dtype == 0)
        embed_scaled_kernel<float><<<T, 256, 0, stream>>>((const int32_t*)ids, (const int32_t*)positions, (const float*)table,
                                                          (const float*)pos_table, (float*)out, d, vocab, max_pos, scale);
    else
        embed_scaled_kernel<bf16_t><<<T, 256, 0, stream>>>((const int32_t*)ids, (const int32_t*)positions, (const bf16_t*)table,
                                                           (const bf16_t*)pos_table, (float*)out, d, vocab, max_pos, scale);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- embedding: row * scale + row of a table of token pairs
// out[t] = table[ids[t]] * scale + pairs[(prev * mul_prev + ids[t] * mul_cur) mod buckets], prev the token before
// ids[t] in its sequence; a sequence's first token (position 0) takes row `buckets`.  The token before the first
// row of a portion is what `last_token[slot]` holds: remember_last_kernel leaves every sequence's last token there
// after the rows have been read (a launch of its own: the first row of a portion must not see it).  `pairs` may be
// null (no second table).  With `freq` (float32 [(d + 1) / 2]) a sinusoid of the position is added: column 2i gets
// sin(position * freq[i]), column 2i + 1 the cosine of the same angle, the angle a float32 product.
template <typename T>
__global__ void embed_pair_hash_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ positions,
                                       const int32_t* __restrict__ seq_of_token, const int32_t* __restrict__ q_start,
                                       const int32_t* __restrict__ state_slot, const int32_t* __restrict__ last_token,
                                       const T* __restrict__ table, const T* __restrict__ pairs, float* __restrict__ out,
                                       int d, int vocab, int buckets, long long mul_prev, long long mul_cur, float scale,
                                       const float* __restrict__ freq) {
    const int t = blockIdx.x;
    const int id = ids[t];
    if (id < 0 || id >= vocab) return;      // unreachable after the host's check
    int row = buckets;
    if (pairs && positions[t] > 0) {
        const int s = seq_of_token[t];
        const int prev = (t == q_start[s]) ? last_token[state_slot[s]] : ids[t - 1];
        long long r = (static_cast<long long>(prev) * mul_prev + static_cast<long long>(id) * mul_cur) % buckets;
        if (r < 0) r += buckets;
        row = static_cast<int>(r);
    }
    const T* erow = table + static_cast<size_t>(id) * d;
    const T* prow = pairs + static_cast<size_t>(row) * d;
    float* o = out + static_cast<size_t>(t) * d;
    const float pos = static_cast<float>(positions[t]);
    // a thread takes the two columns that share an angle: one reduction of the angle serves the sine and the cosine
    for (int p = threadIdx.x; 2 * p < d; p += blockDim.x) {
        const int i = 2 * p;
        const bool two = i + 1 < d;
        float v0 = ld(erow + i) * scale, v1 = two ? ld(erow + i + 1) * scale : 0.f;
        if (pairs) {
            v0 += ld(prow + i);
            if (two) v1 += ld(prow + i + 1);
        }
        if (freq) {
            float sn, cs;
            sincosf(pos * freq[p], &sn, &cs);
            v0 += sn;
            v1 += cs;
        }
        o[i] = v0;
        if (two) o[i + 1] = v1;
    }
}

__global__ void remember_last_kernel(const int32_t* __restrict__ ids, const int32_t* __restrict__ q_start,
                                     const int32_t* __restrict__ q_len, const int32_t* __restrict__ state_slot,
                                     int32_t* __restrict__ last_token, int B) {
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < B && q_len[b] > 0) last_token[state_slot[b]] = ids[q_start[b] + q_len[b] - 1];
}

NI_EXPORT int ni_embed_pair_hash(const void* ids, const void* positions, const void* seq_of_token, const void* q_start,
                                 const void* q_len, const void* state_slot, void* last_token, const void* table,
                                 const void* pairs, void* out, int T, int B, int d, int vocab, int buckets, long long mul_prev,
                                 long long mul_cur, float scale, const void* freq, int dtype, hipStream_t stream) {
    if (T <= 0 || B <= 0) return 0;
    if (pairs && buckets < 1) return -1;
    if (dtype == 0)
        embed_pair_hash_kernel<float><<<T, 256, 0, stream>>>((const int32_t*)ids, (const int32_t*)positions, (const int32_t*)seq_of_token,
            (const int32_t*)q_start, (const int32_t*)state_slot, (const int32_t*)last_token, (const float*)table, (const float*)pairs,
            (float*)out, d, vocab, buckets, mul_prev, mul_cur, scale, (const float*)freq);
    else
        embed_pair_hash_kernel<bf16_t><<<T, 256, 0, stream>>>((const int32_t*)ids, (const int32_t*)positions, (const int32_t*)seq_of_token,
            (const int32_t*)q_start, (const int32_t*)state_slot, (const int32_t*)last_token, (const bf16_t*)table, (const bf16_t*)pairs,
            (float*)out, d, vocab, buckets, mul_prev, mul_cur, scale, (const float*)freq);
    remember_last_kernel<<<blocks_of(B, 64), 64, 0, stream>>>((const int32_t*)ids, (const int32_t*)q_start, (const int32_t*)q_len,
                                                               (const int32_t*)state_slot, (int32_t*)last_token, B);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- h[t, :] += extra[t, :] + vec   (extra may be absent)
__global__ void add_rows_vector_kernel(float* __restrict__ h, const float* __restrict__ extra, const float* __restrict__ vec,
                                       int d, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) h[i] = (extra ? h[i] + extra[i] : h[i]) + vec[i % d];
}

NI_EXPORT int ni_add_rows_vector(void* h, const void* extra, const void* vec, int T, int d, hipStream_t stream) {
    const size_t n = static_cast<size_t>(T) * d;
    if (n == 0) return 0;
    add_rows_vector_kernel<<<blocks_of(n, 256), 256, 0, stream>>>((float*)h, (const float*)extra, (const float*)vec, d, n);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- h[t, :] += vec
__global__ void add_vector_kernel(float* __restrict__ h, const float* __restrict__ vec, int d, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) h[i] += vec[i % d];
}

NI_EXPORT int ni_add_vector(void* h, const void* vec, int T, int d, hipStream_t stream) {
    const size_t n = static_cast<size_t>(T) * d;
    if (n == 0) return 0;
    add_vector_kernel<<<blocks_of(n, 256), 256, 0, stream>>>((float*)h, (const float*)vec, d, n);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- h += (a + b); x = h in the compute type
// a and b (b may be absent) are float32 or the compute type; the two are added first, then the stream.
template <typename TA, typename TB, typename TX>
__global__ void stream_add_kernel(float* __restrict__ h, const TA* __restrict__ a, const TB* __restrict__ b,
                                  TX* __restrict__ x, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    float s = ld(a + i);
    if (b) s += ld(b + i);
    const float v = h[i] + s;
    h[i] = v;
    if (x) st(x + i, v);
}

template <typename TA, typename TB>
static void launch_stream_add(float* h, const TA* a, const TB* b, void* x, int x_dtype, size_t n, hipStream_t stream) {
    const unsigned blocks = blocks_of(n, 256);
    if (x_dtype == 0)
        stream_add_kernel<TA, TB, float><<<blocks, 256, 0, stream>>>(h, a, b, (float*)x, n);
    else
        stream_add_kernel<TA, TB, bf16_t><<<blocks, 256, 0, stream>>>(h, a, b, (bf16_t*)x, n);
}

NI_EXPORT int ni_stream_add(void* h, const void* a, int a_dtype, const void* b, int b_dtype, void* x, int x_dtype,
                            int T, int d, hipStream_t stream) {
    const size_t n = static_cast<size_t>(T) * d;
    if (n == 0) return 0;
    if (a_dtype == 0 && b_dtype == 0) launch_stream_add((float*)h, (const float*)a, (const float*)b, x, x_dtype, n, stream);
    else if (a_dtype == 0) launch_stream_add((float*)h, (const float*)a, (const bf16_t*)b, x, x_dtype, n, stream);
    else if (b_dtype == 0) launch_stream_add((float*)h, (const bf16_t*)a, (const float*)b, x, x_dtype, n, stream);
    else launch_stream_add((float*)h, (const bf16_t*)a, (const bf16_t*)b, x, x_dtype, n, stream);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- g = gelu_tanh(z) * side_row
// z float32 [T, width] (columns beyond `ds` are padding and give zeros); the side row of token t is
// table[ids[t], first : first + ds].
template <typename TT, typename TO>
__global__ void gated_side_kernel(const float* __restrict__ z, const TT* __restrict__ table, const int32_t* __restrict__ ids,
                                  TO* __restrict__ out, int width, int ds, int table_cols, int first, int vocab, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int t = static_cast<int>(i / width), c = static_cast<int>(i % width);
    float v = 0.f;
    const int id = ids[t];
    if (c < ds && id >= 0 && id < vocab)
        v = gelu_tanh_f(z[i]) * ld(table + static_cast<size_t>(id) * table_cols + first + c);
    st(out + i, v);
}

NI_EXPORT int ni_gated_side(const void* z, const void* table, const void* ids, void* out, int T, int width, int ds,
                            int table_cols, int first, int vocab, int dtype, hipStream_t stream) {
    const size_t n = static_cast<size_t>(T) * width;
    if (n == 0) return 0;
    if (dtype == 0)
        gated_side_kernel<float, float><<<blocks_of(n, 256), 256, 0, stream>>>(
            (const float*)z, (const float*)table, (const int32_t*)ids, (float*)out, width, ds, table_cols, first, vocab, n);
    else
        gated_side_kernel<bf16_t, bf16_t><<<blocks_of(n, 256), 256, 0, stream>>>(
            (const float*)z, (const bf16_t*)table, (const int32_t*)ids, (bf16_t*)out, width, ds, table_cols, first, vocab, n);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- h += y / sqrt(mean(y^2) + eps) * w
__global__ void add_rmsnormed_kernel(float* __restrict__ h, const float* __restrict__ y, const float* __restrict__ w,
                                     int d, float eps) {
    __shared__ float scratch[16];
    const size_t base = static_cast<size_t>(blockIdx.x) * d;
    float ss = 0.f;
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = y[base + i];
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) h[base + i] += (y[base + i] * inv) * w[i];
}

NI_EXPORT int ni_add_rmsnormed(void* h, const void* y, const void* w, int T, int d, float eps, hipStream_t stream) {
    if (T <= 0) return 0;
    const int threads = d <= 256 ? 64 : d <= 1024 ? 256 : 512;
    add_rmsnormed_kernel<<<T, threads, 0, stream>>>((float*)h, (const float*)y, (const float*)w, d, eps);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the stream behind a norm: h = rmsnorm(alpha h + sum of addends) * w
// The stream itself takes the normed sum (a block whose norm stands behind the sum); x, if given, is the same in the
// compute type for the products that read it next.  addends float32 [n_addends][T][d], summed in their order and then
// added to alpha * h; all of it float32.  A thread reads in the second pass what it wrote itself in the first.
#define POST_NORM_ITEMS 8       // elements of a row a thread keeps in registers: rows of up to 8 * 512 elements

template <typename X>
__global__ void post_norm_kernel(float* __restrict__ h, const float* __restrict__ addends, int n_addends, size_t addend_stride,
                                 float alpha, const float* __restrict__ w, float eps, X* __restrict__ x, int d) {
    __shared__ float scratch[16];
    const size_t base = static_cast<size_t>(blockIdx.x) * d;
    float ss = 0.f;
    if (d <= POST_NORM_ITEMS * static_cast<int>(blockDim.x)) {
        // the row stays in registers between the sum and the division: every element is read once and written once
        float v[POST_NORM_ITEMS];
#pragma unroll
        for (int u = 0; u < POST_NORM_ITEMS; ++u) {
            const int i = threadIdx.x + u * blockDim.x;
            v[u] = 0.f;
            if (i < d) {
                v[u] = alpha * h[base + i];
                if (n_addends > 0) {
                    float a = addends[base + i];
                    for (int s = 1; s < n_addends; ++s) a += addends[s * addend_stride + base + i];
                    v[u] += a;
                }
                ss += v[u] * v[u];
            }
        }
        const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(d) + eps);
#pragma unroll
        for (int u = 0; u < POST_NORM_ITEMS; ++u) {
            const int i = threadIdx.x + u * blockDim.x;
            if (i < d) {
                const float r = (v[u] * inv) * w[i];
                h[base + i] = r;
                if (x) st(x + base + i, r);
            }
        }
        return;
    }
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        float v = alpha * h[base + i];
        if (n_addends > 0) {
            float a = addends[base + i];
            for (int s = 1; s < n_addends; ++s) a += addends[s * addend_stride + base + i];
            v += a;
        }
        h[base + i] = v;
        ss += v * v;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / static_cast<float>(d) + eps);
    for (int i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = (h[base + i] * inv) * w[i];
        h[base + i] = v;
        if (x) st(x + base + i, v);
    }
}

NI_EXPORT int ni_post_norm(void* h, const void* addends, int n_addends, float alpha, const void* w, float eps, void* x, int x_dtype,
                           int T, int d, hipStream_t stream) {
    if (T <= 0 || d <= 0) return 0;
    if (n_addends < 0 || (n_addends > 0 && !addends)) return -1;
    const int threads = d <= 256 ? 64 : d <= 1024 ? 256 : 512;
    const size_t stride = static_cast<size_t>(T) * d;
    if (x_dtype == 0)
        post_norm_kernel<float><<<T, threads, 0, stream>>>((float*)h, (const float*)addends, n_addends, stride, alpha, (const float*)w, eps,
                                                           (float*)x, d);
    else
        post_norm_kernel<bf16_t><<<T, threads, 0, stream>>>((float*)h, (const float*)addends, n_addends, stride, alpha, (const float*)w, eps,
                                                            (bf16_t*)x, d);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- y = x / sqrt(mean(x^2) + eps) * w over columns of wider rows
// x: n columns of float32 rows of stride `stride` (a product's accumulators); y [T, n] in the type T
template <typename T>
__global__ void rmsnorm_cols_kernel(const float* __restrict__ x, int stride, const float* __restrict__ w, T* __restrict__ y,
                                    int n, float eps) {
    __shared__ float scratch[16];
    const float* row = x + static_cast<size_t>(blockIdx.x) * stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < n; i += blockDim.x) ss += row[i] * row[i];
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(n) + eps);
    for (int i = threadIdx.x; i < n; i += blockDim.x) st(y + static_cast<size_t>(blockIdx.x) * n + i, (row[i] * inv) * w[i]);
}

NI_EXPORT int ni_rmsnorm_cols(const void* x, int stride, const void* w, void* y, int T, int n, float eps, int dtype, hipStream_t stream) {
    if (T <= 0 || n <= 0) return 0;
    if (stride < n) return -1;
    const int threads = n <= 256 ? 64 : n <= 1024 ? 256 : 512;
    if (dtype == 0)
        rmsnorm_cols_kernel<float><<<T, threads, 0, stream>>>((const float*)x, stride, (const float*)w, (float*)y, n, eps);
    else
        rmsnorm_cols_kernel<bf16_t><<<T, threads, 0, stream>>>((const float*)x, stride, (const float*)w, (bf16_t*)y, n, eps);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- a weighted sum of earlier states of the stream
// out[t, :] = sum_j w[j] * hist[j][t, :] for j < n; hist is [n][T][d] float32 (whole streams one after the other)
__global__ void depth_mix_kernel(const float* __restrict__ hist, const float* __restrict__ w, float* __restrict__ out, int n,
                                 size_t per, bool pieces) {
    const size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 4;
    if (i >= per) return;
    if (pieces) {           // whole 16-byte pieces: `per` is a multiple of 4 and both buffers are aligned
        float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int j = 0; j < n; ++j) {
            const float4 v = *reinterpret_cast<const float4*>(hist + static_cast<size_t>(j) * per + i);
            const float wj = w[j];
            acc.x += wj * v.x; acc.y += wj * v.y; acc.z += wj * v.z; acc.w += wj * v.w;
        }
        *reinterpret_cast<float4*>(out + i) = acc;
    } else {
        for (size_t e = i; e < per && e < i + 4; ++e) {
            float acc = 0.f;
            for (int j = 0; j < n; ++j) acc += w[j] * hist[static_cast<size_t>(j) * per + e];
            out[e] = acc;
        }
    }
}

NI_EXPORT int ni_depth_mix(const void* hist, const void* w, void* out, int n, int T, int d, hipStream_t stream) {
    const size_t per = static_cast<size_t>(T) * d;
    if (per == 0 || n <= 0) return 0;
    const bool pieces = per % 4 == 0 && reinterpret_cast<uintptr_t>(hist) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
    depth_mix_kernel<<<blocks_of((per + 3) / 4, 256), 256, 0, stream>>>((const float*)hist, (const float*)w, (float*)out, n, per, pieces);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- a polynomial of normed powers as activation
//   y = a N(z) + b N(z^2) + c N(z^3) + e,   N(u) = u / sqrt(mean(u^2) + eps) over the row, powers element by element
// z float32 [T, n] (a product's accumulators), coef float32 [4] = (a, b, c, e); y in the type T.  A row is taken by
// gridDim.y workgroups, each with its share of the elements (and the whole row's three sums).
template <typename T>
__global__ void __launch_bounds__(256)
poly_norm_kernel(const float* __restrict__ z, const float* __restrict__ coef, T* __restrict__ y, int n, float eps) {
    __shared__ float scratch[16];
    const float* row = z + static_cast<size_t>(blockIdx.x) * n;
    float s2 = 0.f, s4 = 0.f, s6 = 0.f;
    if (n % 4 == 0 && reinterpret_cast<uintptr_t>(z) % 16 == 0) {        // whole 16-byte pieces
        for (int i = 4 * threadIdx.x; i < n; i += 4 * blockDim.x) {
            const float4 q = *reinterpret_cast<const float4*>(row + i);
            const float a = q.x * q.x, b = q.y * q.y, c = q.z * q.z, e = q.w * q.w;
            s2 += (a + b) + (c + e);
            s4 += (a * a + b * b) + (c * c + e * e);
            s6 += (a * a * a + b * b * b) + (c * c * c + e * e * e);
        }
    } else {
        for (int i = threadIdx.x; i < n; i += blockDim.x) {
            const float v = row[i], v2 = v * v;
            s2 += v2;
            s4 += v2 * v2;
            s6 += v2 * v2 * v2;
        }
    }
    s2 = block_sum(s2, scratch);
    s4 = block_sum(s4, scratch);
    s6 = block_sum(s6, scratch);
    const float fn = static_cast<float>(n);
    const float r1 = coef[0] / sqrtf(s2 / fn + eps), r2 = coef[1] / sqrtf(s4 / fn + eps), r3 = coef[2] / sqrtf(s6 / fn + eps);
    const float e = coef[3];
    const int per = (n + gridDim.y - 1) / gridDim.y;
    for (int i = blockIdx.y * per + threadIdx.x; i < min(n, (blockIdx.y + 1) * per); i += blockDim.x) {
        const float v = row[i];
        st(y + static_cast<size_t>(blockIdx.x) * n + i, (v * r1 + (v * v) * r2) + ((v * v * v) * r3 + e));
    }
}

NI_EXPORT int ni_poly_norm(const void* z, const void* coef, void* y, int T, int n, float eps, int dtype, hipStream_t stream) {
    if (T <= 0 || n <= 0) return 0;
    const dim3 grid(T, T >= 64 ? 1 : std::max(1, std::min(16, (n + 1023) / 1024)));
    if (dtype == 0)
        poly_norm_kernel<float><<<grid, 256, 0, stream>>>((const float*)z, (const float*)coef, (float*)y, n, eps);
    else
        poly_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)z, (const float*)coef, (bf16_t*)y, n, eps);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- x *= s, element by element (float32)
__global__ void scale_kernel(float* __restrict__ x, float s, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i < n) x[i] *= s;
}

NI_EXPORT int ni_scale(void* x, float s, size_t n, hipStream_t stream) {
    if (n == 0) return 0;
    scale_kernel<<<blocks_of(n, 256), 256, 0, stream>>>((float*)x, s, n);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- read-outs head by head times a gate
//   y[t, h * dv + c] = o[h][t][c] * sigmoid(g[t, (h * dv + c) / per])      o float32 [H][T][dv], g float32 rows of stride
//   g_stride; per = 1: a gate a channel, per = dv: a gate a head
template <typename T>
__global__ void gate_heads_kernel(const float* __restrict__ o, const float* __restrict__ g, int g_stride, T* __restrict__ y,
                                  int Tn, int H, int dv, int per, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = static_cast<int>(i % dv), h = static_cast<int>((i / dv) % H);
    const size_t t = i / (static_cast<size_t>(dv) * H);
    const float gate = 1.0f / (1.0f + expf(-g[t * g_stride + (h * dv + c) / per]));
    st(y + i, o[(static_cast<size_t>(h) * Tn + t) * dv + c] * gate);
}

NI_EXPORT int ni_gate_heads(const void* o, const void* g, int g_stride, void* y, int T, int H, int dv, int per, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * H * dv;
    if (total == 0) return 0;
    if (per < 1 || g_stride < (H * dv + per - 1) / per) return -1;
    if (dtype == 0)
        gate_heads_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)o, (const float*)g, g_stride, (float*)y, T, H, dv, per, total);
    else
        gate_heads_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)o, (const float*)g, g_stride, (bf16_t*)y, T, H, dv, per, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- rows of heads, token by token, as heads of rows
//   y[h][t][c] = x[t, h * n + c]      (what a product per head reads: every head's rows together)
template <typename T>
__global__ void heads_apart_kernel(const T* __restrict__ x, int x_stride, T* __restrict__ y, int Tn, int H, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = static_cast<int>(i % n);
    const size_t t = (i / n) % Tn;
    const int h = static_cast<int>(i / (static_cast<size_t>(n) * Tn));
    y[i] = x[t * x_stride + h * n + c];
}

NI_EXPORT int ni_heads_apart(const void* x, int x_stride, void* y, int T, int H, int n, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * H * n;
    if (total == 0) return 0;
    if (x_stride < H * n) return -1;
    if (dtype == 0)
        heads_apart_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)x, x_stride, (float*)y, T, H, n, total);
    else
        heads_apart_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const bf16_t*)x, x_stride, (bf16_t*)y, T, H, n, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- rows times the sigmoid of a gate
//   y[t, j] = x[t, j] * sigmoid(g[t, j / per])      x [T, n] in the compute type, g float32 rows of stride g_stride;
//   per = 1: a gate a channel, per = a head's channels: a gate a head
template <typename T>
__global__ void gate_rows_kernel(const T* __restrict__ x, const float* __restrict__ g, int g_stride, T* __restrict__ y, int n,
                                 int per, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const size_t t = i / n;
    const int j = static_cast<int>(i % n);
    const float gate = 1.0f / (1.0f + expf(-g[t * g_stride + j / per]));
    st(y + i, ld(x + i) * gate);
}

NI_EXPORT int ni_gate_rows(const void* x, const void* g, int g_stride, void* y, int T, int n, int per, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(T) * n;
    if (total == 0) return 0;
    if (per < 1 || g_stride < (n + per - 1) / per) return -1;
    if (dtype == 0)
        gate_rows_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)x, (const float*)g, g_stride, (float*)y, n, per, total);
    else
        gate_rows_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const bf16_t*)x, (const float*)g, g_stride, (bf16_t*)y, n, per, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- pages of a pool, picked through a block table
//   out[i] = pool[table[pairs[2 i] * width + pairs[2 i + 1]]]      a page is `page_elems` contiguous elements; a page the
//   table does not hold (< 0) gives zeros
template <typename T>
__global__ void gather_pages_kernel(const T* __restrict__ pool, const int32_t* __restrict__ table, int width,
                                    const int32_t* __restrict__ pairs, T* __restrict__ out, int page_elems) {
    const int i = blockIdx.x;
    const int page = table[static_cast<size_t>(pairs[2 * i]) * width + pairs[2 * i + 1]];
    const T* src = pool + static_cast<size_t>(max(page, 0)) * page_elems;
    T* dst = out + static_cast<size_t>(i) * page_elems;
    for (int e = threadIdx.x; e < page_elems; e += blockDim.x) st(dst + e, page >= 0 ? ld(src + e) : 0.f);
}

NI_EXPORT int ni_gather_pages(const void* pool, const void* table, int width, const void* pairs, void* out, int n_pages,
                              int page_elems, int dtype, hipStream_t stream) {
    if (n_pages <= 0 || page_elems <= 0) return 0;
    if (width < 1) return -1;
    if (dtype == 0)
        gather_pages_kernel<float><<<n_pages, 256, 0, stream>>>((const float*)pool, (const int32_t*)table, width, (const int32_t*)pairs,
                                                                (float*)out, page_elems);
    else
        gather_pages_kernel<bf16_t><<<n_pages, 256, 0, stream>>>((const bf16_t*)pool, (const int32_t*)table, width, (const int32_t*)pairs,
                                                                 (bf16_t*)out, page_elems);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- rows of heads, page by page, as pages of heads
//   y[p][h][s][c] = x[(p * page + s), h * n + c]      (the layout of a pool of keys or values: [page][head][slot][channel])
template <typename T>
__global__ void rows_to_pages_kernel(const T* __restrict__ x, T* __restrict__ y, int page, int H, int n, size_t total) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= total) return;
    const int c = static_cast<int>(i % n);
    const int s = static_cast<int>((i / n) % page);
    const int h = static_cast<int>((i / (static_cast<size_t>(n) * page)) % H);
    const size_t p = i / (static_cast<size_t>(n) * page * H);
    y[i] = x[(p * page + s) * (static_cast<size_t>(H) * n) + h * n + c];
}

NI_EXPORT int ni_rows_to_pages(const void* x, void* y, int n_pages, int page, int H, int n, int dtype, hipStream_t stream) {
    const size_t total = static_cast<size_t>(n_pages) * page * H * n;
    if (total == 0) return 0;
    if (dtype == 0)
        rows_to_pages_kernel<float><<<blocks_of(total, 256), 256, 0, stream>>>((const float*)x, (float*)y, page, H, n, total);
    else
        rows_to_pages_kernel<bf16_t><<<blocks_of(total, 256), 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)y, page, H, n, total);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the router's choice
// z float32 [T, E]: the `top` experts of a row with the largest scores (the lower index on equal scores) and their weights.
// `scoring` says what an expert's value is and how the chosen ones are weighed:
//   0  the logit; weights: the softmax among the chosen
//   1  the logit; weights: the softmax over all E experts, not renormalised
//   2  sigmoid(logit); weights: the values themselves, not renormalised
// every weight times `route_scale`.  An expert is chosen by its value plus `correction[e]` (float32 [E]; null: the value
// alone); the weights never see the correction.
// With `n_groups` > 1 the experts form that many equal groups of neighbours; a group counts as much as the sum of its
// `group_top` largest scores (1: its largest score), and only experts of the `keep` best groups (the lower index on
// equal ones) can be chosen: the others' scores count as minus infinity.
// chosen int32 [T, top], mix float32 [T, top], and (if asked for) the same as a row over all experts, zero where
// an expert was not chosen.
// One wavefront a row.  More than 64 experts: a lane keeps the scores of experts lane, lane + 64, ...; each round finds
// the largest score not yet taken (the lowest index among equal ones) by two butterflies over the lanes.  Up to 64
// experts: `route_top_lanes_kernel` below, which ranks instead of searching.
#define NO_EXPERT 0x7fffffff

__device__ __forceinline__ int lowest_of(int cand) {
#pragma unroll
    for (int off = WAVE / 2; off > 0; off >>= 1) cand = min(cand, __shfl_xor(cand, off, WAVE));
    return cand;
}

template <int SLOTS>
__global__ void route_top_kernel(const float* __restrict__ z, const float* __restrict__ correction, int32_t* __restrict__ chosen,
                                 float* __restrict__ mix, float* __restrict__ mix_all, int T, int E, int top, int scoring,
                                 int n_groups, int keep, int group_top, float route_scale) {
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* row = z + static_cast<size_t>(t) * E;
    int32_t* c = chosen + static_cast<size_t>(t) * top;
    float* m = mix + static_cast<size_t>(t) * top;
    // the row once, into registers: slot j of a lane is expert lane + 64 j (every round below would else wait for memory
    // again); a logit that is no number is never preferred.  vals: what chooses; raw: what weighs
    float vals[SLOTS], raw[SLOTS];
#pragma unroll
    for (int j = 0; j < SLOTS; ++j) {
        const int e = lane + j * WAVE;
        float ze = e < E ? row[e] : -INFINITY;
        if (!(ze == ze)) ze = -INFINITY;
        raw[j] = scoring == 2 ? 1.0f / (1.0f + expf(-ze)) : ze;
        vals[j] = e < E ? raw[j] + (correction ? correction[e] : 0.f) : -INFINITY;
    }
    if (mix_all) {                  // zeros first; the fence lets them land before lane 0 writes the chosen ones at the end
        for (int e = lane; e < E; e += WAVE) mix_all[static_cast<size_t>(t) * E + e] = 0.f;
        __threadfence_block();
    }
    unsigned long long open_groups = ~0ull;       // bit g: experts of group g may be chosen
    const int per_group = E / max(n_groups, 1);
    if (n_groups > 1) {
        // lane g ends up with the score of group g: the sum of its `group_top` largest scores
        float mine = -INFINITY;
        for (int g = 0; g < n_groups; ++g) {
            float sum = 0.f;
            unsigned used = 0;      // bit j: this lane's expert lane + 64 j has been counted for this group
            for (int n = 0; n < group_top; ++n) {
                float v = -INFINITY;
                int at = NO_EXPERT;
#pragma unroll
                for (int j = 0; j < SLOTS; ++j) {
                    const int e = lane + j * WAVE;
                    if (e < E && e / per_group == g && !((used >> j) & 1u) && (at == NO_EXPERT || vals[j] > v)) { at = e; v = vals[j]; }
                }
                const float vmax = wave_max(v);
                const int cand = lowest_of((at != NO_EXPERT && v == vmax) ? at : NO_EXPERT);
                if (cand == NO_EXPERT) break;             // a group of fewer experts than group_top (the same for all lanes)
                if (cand % WAVE == lane) used |= 1u << (cand / WAVE);
                sum += vmax;
            }
            if (lane == g) mine = sum;
        }
        open_groups = 0ull;
        bool used = lane >= n_groups;
        for (int k = 0; k < keep; ++k) {
            const float v = used ? -INFINITY : mine;
            const float vmax = wave_max(v);
            const int cand = lowest_of((!used && v == vmax) ? lane : NO_EXPERT);
            if (cand == NO_EXPERT) break;         // unreachable: keep <= n_groups
            if (cand == lane) used = true;
            open_groups |= 1ull << cand;
        }
    }
    float best = 0.f, total = 1.f;
    if (scoring == 1) {             // the softmax runs over every expert, chosen or not
        float v = -INFINITY;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) v = fmaxf(v, raw[j]);
        best = wave_max(v);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j)
            if (lane + j * WAVE < E && raw[j] > -INFINITY) sum += expf(raw[j] - best);
        total = wave_sum(sum);
    }
    unsigned taken_mask = 0;        // bit j: this lane's expert lane + 64 j has been chosen
    // up to 64 chosen experts stay in registers, the k-th in lane k; more go through the result's own memory
    const bool in_lanes = top <= WAVE;
    int my_expert = 0;
    float my_value = -INFINITY;
    for (int k = 0; k < top; ++k) {
        float v = -INFINITY;
        int at = NO_EXPERT;
#pragma unroll
        for (int j = 0; j < SLOTS; ++j) {
            const int e = lane + j * WAVE;
            if (e >= E) continue;
            const bool taken = (taken_mask >> j) & 1u;
            const bool open = (open_groups >> (n_groups > 1 ? e / per_group : 0)) & 1ull;
            if (!taken && open && (at == NO_EXPERT || vals[j] > v)) { at = e; v = vals[j]; }
        }
        const float vmax = wave_max(v);
        const int cand = lowest_of((at != NO_EXPERT && v == vmax) ? at : NO_EXPERT);
        if (cand % WAVE == lane) taken_mask |= 1u << (cand / WAVE);
        float mine = 0.f;           // what weighs the chosen expert: only its owner has it
#pragma unroll
        for (int j = 0; j < SLOTS; ++j)
            if (lane + j * WAVE == cand) mine = raw[j];
        const float value = wave_sum(mine);
        if (in_lanes) {
            if (lane == k) { my_expert = cand; my_value = value; }
        } else if (lane == 0) {
            c[k] = cand;
            m[k] = value;
        }
    }
    if (in_lanes) {
        if (scoring == 0) {         // the softmax among the chosen
            best = wave_max(my_value);
            total = wave_sum(lane < top ? expf(my_value - best) : 0.f);
        }
        if (lane < top) {
            const float w = (scoring == 2 ? my_value : expf(my_value - best) / total) * route_scale;
            c[lane] = my_expert;
            m[lane] = w;
            if (mix_all) mix_all[static_cast<size_t>(t) * E + my_expert] = w;
        }
        return;
    }
    if (lane == 0) {
        if (scoring == 0) {         // the softmax among the chosen
            best = -INFINITY;
            for (int k = 0; k < top; ++k) best = fmaxf(best, m[k]);
            total = 0.f;
            for (int k = 0; k < top; ++k) total += expf(m[k] - best);
        }
        for (int k = 0; k < top; ++k) {
            const float w = (scoring == 2 ? m[k] : expf(m[k] - best) / total) * route_scale;
            m[k] = w;
            if (mix_all) mix_all[static_cast<size_t>(t) * E + c[k]] = w;
        }
    }
}

// The same for up to 64 experts, one a lane, without butterflies: a lane ranks its expert among the others by walking
// the E lanes' values (each read into a scalar register, `lane_value`; a lone wavefront's time is its instructions,
// so the walks stop at E), first inside its group (which experts count
// for the group's score), then its group among the groups, then its expert among those that may be chosen; the
// expert of rank k is the k-th choice.  Better is: the larger score, or of equal scores the lower index, as above.
__device__ __forceinline__ float lane_value(float v, int j) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), j)); }
__device__ __forceinline__ int lane_value(int v, int j) { return __builtin_amdgcn_readlane(v, j); }
__device__ __forceinline__ bool better(float a, int ia, float b, int ib) { return a > b || (a == b && ia < ib); }

__global__ void __launch_bounds__(WAVE)
route_top_lanes_kernel(const float* __restrict__ z, const float* __restrict__ correction, int32_t* __restrict__ chosen,
                       float* __restrict__ mix, float* __restrict__ mix_all, int E, int top, int scoring, int n_groups, int keep,
                       int group_top, float route_scale) {
    const int t = blockIdx.x, e = threadIdx.x;
    const bool mine = e < E;
    float ze = mine ? z[static_cast<size_t>(t) * E + e] : -INFINITY;
    if (!(ze == ze)) ze = -INFINITY;                  // a logit that is no number is never preferred
    const float raw = scoring == 2 ? 1.0f / (1.0f + expf(-ze)) : ze;
    const float val = mine ? raw + (correction ? correction[e] : 0.f) : -INFINITY;
    bool open = mine;
    if (n_groups > 1) {
        const int per_group = E / n_groups;
        const int grp = mine ? e / per_group : -1;
        int in_group = 0;                             // experts of my group that are better than mine
        for (int j = 0; j < E; ++j)
            in_group += (lane_value(grp, j) == grp && better(lane_value(val, j), j, val, e)) ? 1 : 0;
        const float counted = (mine && in_group < group_top) ? val : 0.f;
        float score = 0.f;                            // of my group: the sum of its `group_top` best scores
        for (int j = 0; j < E; ++j)
            score += lane_value(grp, j) == grp ? lane_value(counted, j) : 0.f;
        const int first = (mine && e % per_group == 0) ? grp : -1;      // a group's first lane speaks for it
        int ahead = 0;                                // groups that are better than mine
        for (int j = 0; j < E; ++j) {
            const int gj = lane_value(first, j);
            ahead += (gj >= 0 && better(lane_value(score, j), gj, score, grp)) ? 1 : 0;
        }
        open = mine && ahead < keep;
    }
    const unsigned long long open_mask = __ballot(open);
    int rank = 0;                                     // experts that may be chosen and are better than mine
    for (int j = 0; j < E; ++j)
        rank += (((open_mask >> j) & 1ull) && better(lane_value(val, j), j, val, e)) ? 1 : 0;
    const bool taken = open && rank < top;
    const unsigned long long taken_mask = __ballot(taken);
    float w = raw;
    if (scoring != 2) {
        const unsigned long long over = scoring == 1 ? __ballot(mine) : taken_mask;     // what the softmax runs over
        float best = -INFINITY, total = 0.f;
        for (int j = 0; j < E; ++j)
            if ((over >> j) & 1ull) best = fmaxf(best, lane_value(raw, j));
        const float mine_exp = raw > -INFINITY ? expf(raw - best) : 0.f;
        for (int j = 0; j < E; ++j)
            if ((over >> j) & 1ull) total += lane_value(mine_exp, j);
        w = mine_exp / total;
    }
    w *= route_scale;
    if (taken) {
        chosen[static_cast<size_t>(t) * top + rank] = e;
        mix[static_cast<size_t>(t) * top + rank] = w;
    }
    if (mix_all && mine) mix_all[static_cast<size_t>(t) * E + e] = taken ? w : 0.f;
}

NI_EXPORT int ni_route_top(const void* z, const void* correction, void* chosen, void* mix, void* mix_all, int T, int E, int top,
                           int scoring, int n_groups, int keep, int group_top, float route_scale, hipStream_t stream) {
    if (T <= 0) return 0;
    if (top < 1 || top > E || E > 32 * WAVE || scoring < 0 || scoring > 2 || group_top < 1) return -1;
    if (n_groups < 1 || n_groups > WAVE || E % n_groups || keep < 1 || keep > n_groups || top > E / n_groups * keep) return -1;
    if (E <= WAVE)
        route_top_lanes_kernel<<<T, WAVE, 0, stream>>>((const float*)z, (const float*)correction, (int32_t*)chosen, (float*)mix,
                                                       (float*)mix_all, E, top, scoring, n_groups, keep, group_top, route_scale);
    else if (E <= 4 * WAVE)
        route_top_kernel<4><<<T, WAVE, 0, stream>>>((const float*)z, (const float*)correction, (int32_t*)chosen, (float*)mix,
                                                    (float*)mix_all, T, E, top, scoring, n_groups, keep, group_top, route_scale);
    else
        route_top_kernel<32><<<T, WAVE, 0, stream>>>((const float*)z, (const float*)correction, (int32_t*)chosen, (float*)mix,
                                                     (float*)mix_all, T, E, top, scoring, n_groups, keep, group_top, route_scale);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- all experts at once, for many rows
// act[t, e * ff + i] = mix_all[t, e] * relu(up[t, e * ff + i])^2 : an expert that was not chosen gives
// zeros, and the product with the experts' down matrices laid side by side is the weighted sum.
template <typename T>
__global__ void experts_act_kernel(const T* __restrict__ up, const float* __restrict__ mix_all, T* __restrict__ act,
                                   int E, int ff, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t width = static_cast<size_t>(E) * ff;
    const size_t t = i / width;
    const int e = static_cast<int>((i % width) / ff);
    const float w = mix_all[t * E + e];
    float v = 0.f;
    if (w != 0.f) {
        const float u = fmaxf(ld(up + i), 0.f);
        v = w * (u * u);
    }
    st(act + i, v);
}

// the same, eight neighbouring elements a thread (ff a multiple of 8: they are one expert's); the elements of an
// expert that was not chosen are not read at all
template <typename T>
__global__ void experts_act_vec_kernel(const T* __restrict__ up, const float* __restrict__ mix_all, T* __restrict__ act,
                                       int E, int ff, size_t pieces) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= pieces) return;
    const size_t i = idx * 8;
    const size_t width = static_cast<size_t>(E) * ff;
    const size_t t = i / width;
    const int e = static_cast<int>((i - t * width) / ff);
    const float w = mix_all[t * E + e];
    float v[8];
    if (w != 0.f) {
        VecIO<T, 8>::load(up + i, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float u = fmaxf(v[j], 0.f);
            v[j] = w * (u * u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = 0.f;
    }
    VecIO<T, 8>::store(act + i, v);
}

// What a gated hidden unit gives from its gate g and its up value u.  `form` 1: silu(g) * u.  `form` 2, the capped form:
// g <- min(g, limit), u <- clamp(u, -limit, limit), then g * sigmoid(slope * g) * (u + 1).
struct GluForm {
    int form;
    float limit, slope;
};

__device__ __forceinline__ float glu_value(float g, float u, const GluForm f) {
    if (f.form == 2) {
        g = fminf(g, f.limit);
        u = fminf(fmaxf(u, -f.limit), f.limit);
        return g / (1.0f + expf(-f.slope * g)) * (u + 1.0f);
    }
    return g / (1.0f + expf(-g)) * u;
}

// the gated forms: an expert's rows of `up` are [gate: ff | up: ff], act[t, e * ff + i] = mix_all[t, e] * glu(gate, up);
// a null mix_all: every expert counts once (one feed-forward that every token uses is E = 1 of these)
template <typename T>
__global__ void experts_act_gated_kernel(const T* __restrict__ up, const float* __restrict__ mix_all, T* __restrict__ act,
                                         int E, int ff, size_t n, GluForm form) {
    const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const size_t width = static_cast<size_t>(E) * ff;
    const size_t t = i / width;
    const int e = static_cast<int>((i % width) / ff), c = static_cast<int>(i % ff);
    const float w = mix_all ? mix_all[t * E + e] : 1.f;
    float v = 0.f;
    if (w != 0.f) {
        const T* src = up + (t * E + e) * 2 * static_cast<size_t>(ff);
        v = w * glu_value(ld(src + c), ld(src + ff + c), form);
    }
    st(act + i, v);
}

// the same, eight neighbouring elements a thread (ff a multiple of 8: they are one expert's); the elements of an
// expert that was not chosen are not read at all
template <typename T>
__global__ void experts_act_gated_vec_kernel(const T* __restrict__ up, const float* __restrict__ mix_all, T* __restrict__ act,
                                             int E, int ff, size_t pieces, GluForm form) {
    const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (idx >= pieces) return;
    const size_t i = idx * 8;
    const size_t width = static_cast<size_t>(E) * ff;
    const size_t t = i / width;
    const size_t in_row = i - t * width;
    const int e = static_cast<int>(in_row / ff), c = static_cast<int>(in_row - static_cast<size_t>(e) * ff);
    const float w = mix_all ? mix_all[t * E + e] : 1.f;
    float v[8];
    if (w != 0.f) {
        const T* src = up + (t * E + e) * 2 * static_cast<size_t>(ff) + c;
        float g[8], u[8];
        VecIO<T, 8>::load(src, g);
        VecIO<T, 8>::load(src + ff, u);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = w * glu_value(g[j], u[j], form);
    } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = 0.f;
    }
    VecIO<T, 8>::store(act + i, v);
}

// `gated` 0: relu(up)^2; 1: silu(gate) * up; 2: the capped form with `limit` and `slope` (see glu_value)
NI_EXPORT int ni_experts_act(const void* up, const void* mix_all, void* act, int T, int E, int ff, int gated, float limit, float slope,
                             int dtype, hipStream_t stream) {
    const size_t n = static_cast<size_t>(T) * E * ff;
    if (n == 0) return 0;
    if (gated < 0 || gated > 2 || (!gated && !mix_all)) return -1;
    const GluForm form{gated, limit, slope};
    if (gated && ff % 8 == 0 && aligned16(up, act)) {
        const size_t pieces = n / 8;
        if (dtype == 0)
            experts_act_gated_vec_kernel<float><<<blocks_of(pieces, 256), 256, 0, stream>>>((const float*)up, (const float*)mix_all, (float*)act, E, ff, pieces, form);
        else
            experts_act_gated_vec_kernel<bf16_t><<<blocks_of(pieces, 256), 256, 0, stream>>>((const bf16_t*)up, (const float*)mix_all, (bf16_t*)act, E, ff, pieces, form);
        return NI_LAUNCH_RESULT();
    }
    if (gated) {
        if (dtype == 0)
            experts_act_gated_kernel<float><<<blocks_of(n, 256), 256, 0, stream>>>((const float*)up, (const float*)mix_all, (float*)act, E, ff, n, form);
        else
            experts_act_gated_kernel<bf16_t><<<blocks_of(n, 256), 256, 0, stream>>>((const bf16_t*)up, (const float*)mix_all, (bf16_t*)act, E, ff, n, form);
        return NI_LAUNCH_RESULT();
    }
    if (ff % 8 == 0 && aligned16(up, act)) {
        const size_t pieces = n / 8;
        if (dtype == 0)
            experts_act_vec_kernel<float><<<blocks_of(pieces, 256), 256, 0, stream>>>((const float*)up, (const float*)mix_all, (float*)act, E, ff, pieces);
        else
            experts_act_vec_kernel<bf16_t><<<blocks_of(pieces, 256), 256, 0, stream>>>((const bf16_t*)up, (const float*)mix_all, (bf16_t*)act, E, ff, pieces);
        return NI_LAUNCH_RESULT();
    }
    if (dtype == 0)
        experts_act_kernel<float><<<blocks_of(n, 256), 256, 0, stream>>>((const float*)up, (const float*)mix_all, (float*)act, E, ff, n);
    else
        experts_act_kernel<bf16_t><<<blocks_of(n, 256), 256, 0, stream>>>((const bf16_t*)up, (const float*)mix_all, (bf16_t*)act, E, ff, n);
    return NI_LAUNCH_RESULT();
}

// ---------------------------------------------------------------- the chosen experts alone, for few rows
// Only the matrices of the chosen experts are read, each row of a matrix by one wavefront: its lanes
// take neighbouring pieces of the row, so a row streams from memory in whole lines.
//   hid[t * top + k, i] = relu(W_up[chosen[t, k] * ff + i, :] . x[t, :])^2        (float32)
//   out[t, r] = sum_k mix[t, k] * W_down[r, chosen[t, k] * ff : +ff] . hid[t * top + k, :]
// A wavefront takes R neighbouring rows at once, with a sum of its own for each: the loads of the R rows are in
// flight together, and the input row is read once for all of them.
template <typename T, int R, bool GATED>
__global__ void experts_up_few_kernel(const T* __restrict__ x, const T* __restrict__ w_up, const int32_t* __restrict__ chosen,
                                      float* __restrict__ hid, int d, int ff, int top, bool vec, GluForm form) {
    // GATED: an expert owns 2 ff rows of w_up, its gate rows and then its up rows; hid = glu(gate . x, up . x)
    const int pair = blockIdx.x;                 // t * top + k
    const int t = pair / top;
    const int e = chosen[pair];
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
    const T* xr = x + static_cast<size_t>(t) * d;
    const int i0 = (blockIdx.y * waves + wave) * R;
    if (i0 >= ff) return;
    constexpr int RR = GATED ? 2 * R : R;        // rows of the matrix a wavefront walks: R, or R gate rows and R up rows
    const T* wr[RR];
#pragma unroll
    for (int u = 0; u < R; ++u) {
        const size_t first = static_cast<size_t>(e) * (GATED ? 2 * ff : ff) + min(i0 + u, ff - 1);
        wr[u] = w_up + first * d;
        if constexpr (GATED) wr[R + u] = w_up + (first + ff) * d;
    }
    float s[RR];
#pragma unroll
    for (int u = 0; u < RR; ++u) s[u] = 0.f;
    if (vec) {          // eight elements a lane and load: a wavefront takes 512 neighbouring elements of a row at once
        for (int c = lane * 8; c < d; c += WAVE * 8) {
            float wv[RR][8], xv[8];
#pragma unroll
            for (int u = 0; u < RR; ++u) VecIO<T, 8>::load(wr[u] + c, wv[u]);
            VecIO<T, 8>::load(xr + c, xv);
#pragma unroll
            for (int u = 0; u < RR; ++u)
#pragma unroll
                for (int j = 0; j < 8; ++j) s[u] += wv[u][j] * xv[j];
        }
    } else {
        for (int c = lane; c < d; c += WAVE) {
            const float xv = ld(xr + c);
#pragma unroll
            for (int u = 0; u < RR; ++u) s[u] += ld(wr[u] + c) * xv;
        }
    }
#pragma unroll
    for (int u = 0; u < RR; ++u) s[u] = wave_sum(s[u]);
#pragma unroll
    for (int u = 0; u < R; ++u) {
        if (lane == 0 && i0 + u < ff) {
            float a;
            if constexpr (GATED) {
                a = glu_value(s[u], s[R + u], form);
            } else {
                a = fmaxf(s[u], 0.f);
                a = a * a;
            }
            hid[static_cast<size_t>(pair) * ff + i0 + u] = a;
        }
    }
}

template <typename T, int R>
__global__ void experts_down_few_kernel(const float* __restrict__ hid, const T* __restrict__ w_down,
                                        const int32_t* __restrict__ chosen, const float* __restrict__ mix,
                                        float* __restrict__ out, int d, int ff, int E, int top, bool vec) {
    const int t = blockIdx.x;
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, waves = blockDim.x / WAVE;
    const int r0 = (blockIdx.y * waves + wave) * R;
    if (r0 >= d) return;
    const size_t row_stride = static_cast<size_t>(E) * ff;
    float total[R];
#pragma unroll
    for (int u = 0; u < R; ++u) total[u] = 0.f;
    for (int k = 0; k < top; ++k) {
        const int e = chosen[t * top + k];
        const float* hr = hid + (static_cast<size_t>(t) * top + k) * ff;
        const T* wr[R];
#pragma unroll
        for (int u = 0; u < R; ++u) wr[u] = w_down + static_cast<size_t>(min(r0 + u, d - 1)) * row_stride + static_cast<size_t>(e) * ff;
        float s[R];
#pragma unroll
        for (int u = 0; u < R; ++u) s[u] = 0.f;
        if (vec) {
            for (int c = lane * 8; c < ff; c += WAVE * 8) {
                float wv[R][8], hv[8];
#pragma unroll
                for (int u = 0; u < R; ++u) VecIO<T, 8>::load(wr[u] + c, wv[u]);
                VecIO<float, 8>::load(hr + c, hv);
#pragma unroll
                for (int u = 0; u < R; ++u)
#pragma unroll
                    for (int j = 0; j < 8; ++j) s[u] += wv[u][j] * hv[j];
            }
        } else {
            for (int c = lane; c < ff; c += WAVE) {
                const float hv = hr[c];
#pragma unroll
                for (int u = 0; u < R; ++u) s[u] += ld(wr[u] + c) * hv;
            }
        }
        const float weight = mix[t * top + k];
#pragma unroll
        for (int u = 0; u < R; ++u) total[u] += weight * wave_sum(s[u]);
    }
    if (lane == 0) {
#pragma unroll
        for (int u = 0; u < R; ++u)
            if (r0 + u < d) out[static_cast<size_t>(t) * d + r0 + u] = total[u];
    }
}

template <typename T, int R>
static void launch_experts_few(const void* x, const void* w_up, const void* w_down, const void* chosen, const void* mix,
                               void* hid, void* out, int T_, int d, int ff, int E, int top, GluForm form, bool vec_up, bool vec_down,
                               hipStream_t stream) {
    const bool gated = form.form != 0;
    constexpr int rows = 4 * R;                  // four wavefronts a workgroup
    dim3 g1(T_ * top, (ff + rows - 1) / rows), g2(T_, (d + rows - 1) / rows);
    if (gated)
        experts_up_few_kernel<T, R, true><<<g1, 256, 0, stream>>>((const T*)x, (const T*)w_up, (const int32_t*)chosen, (float*)hid, d, ff, top, vec_up, form);
    else
        experts_up_few_kernel<T, R, false><<<g1, 256, 0, stream>>>((const T*)x, (const T*)w_up, (const int32_t*)chosen, (float*)hid, d, ff, top, vec_up, form);
    experts_down_few_kernel<T, R><<<g2, 256, 0, stream>>>((const float*)hid, (const T*)w_down, (const int32_t*)chosen,
                                                          (const float*)mix, (float*)out, d, ff, E, top, vec_down);
}

// `gated` 0: w_up [E * ff, d], hid = relu(.)^2; 1 or 2: w_up [E * 2 ff, d] (an expert's gate rows, then its up rows),
// hid = silu(gate) * up, or the capped form with `limit` and `slope` (see glu_value)
NI_EXPORT int ni_experts_few(const void* x, const void* w_up, const void* w_down, const void* chosen, const void* mix,
                             void* hid, void* out, int T, int d, int ff, int E, int top, int gated, float limit, float slope,
                             int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (gated < 0 || gated > 2) return -1;
    // rows of whole 16-byte (bfloat16) or 32-byte (float32) pieces that start on such a piece are read in pieces
    const bool vec_up = d % 8 == 0 && aligned16(x, w_up);
    const bool vec_down = ff % 8 == 0 && aligned16(w_down, hid);
    // four rows a wavefront where that still leaves the second kernel a workgroup for every compute unit, else two
    // (the gated form walks twice the rows in its first kernel and keeps to two)
    const bool four = !gated && static_cast<long long>(T) * ((d + 15) / 16) >= 256;
    const GluForm g{gated, limit, slope};
    if (dtype == 0) {
        if (four) launch_experts_few<float, 4>(x, w_up, w_down, chosen, mix, hid, out, T, d, ff, E, top, g, vec_up, vec_down, stream);
        else launch_experts_few<float, 2>(x, w_up, w_down, chosen, mix, hid, out, T, d, ff, E, top, g, vec_up, vec_down, stream);
    } else {
        if (four) launch_experts_few<bf16_t, 4>(x, w_up, w_down, chosen, mix, hid, out, T, d, ff, E, top, g, vec_up, vec_down, stream);
        else launch_experts_few<bf16_t, 2>(x, w_up, w_down, chosen, mix, hid, out, T, d, ff, E, top, g, vec_up, vec_down, stream);
    }
    return NI_LAUNCH_RESULT();
}
