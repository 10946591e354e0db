// Causal softmax attention over the paged cache with a bias by distance and a query temperature,
// keys and values of different sizes, for gfx950.
//
//     score(i, j) = (q_i . k_j) * scale * temp(i) + bias[i - j, head]      for j <= i
//     temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1)
//
// `bias` is a float32 table [distances, heads] that the host has laid out from the learned rows (one
// row for every distance up to the model's last position), so the kernel needs no logarithm a score.
// Pools are [page, kv_head, slot_in_page, size] with size dk for keys and dv for values.
//
// A window (`window` > 0) narrows what a query sees to its last `window` keys, its own among them, plus the
// first `keep_first` keys of its sequence, which stay visible for good: j <= i and (i - j < window or j < keep_first).
// The kernels then walk only the tiles of 64 keys that hold such keys: the tiles of the kept first keys, then the
// tiles from the one in which the window of the tile's first token starts (`KeyWalk`).  `out_scale` multiplies the
// normalised output (a mixer that is one of several side by side has a weight of its own).
//
// A sink (`sink`, float32 [heads], or null) is one more term exp(sink[head]) in a row's denominator, with no key and
// no value: the weights of a row then sum to less than one.  It counts once a row, whatever the number of runs: the
// kernels add it when a row is finished (a row in runs: when the runs are merged).
//
// One workgroup of four wavefronts takes a tile of consecutive tokens of one sequence and (a chunk of)
// the query heads of one kv head: 16 rows of (token, head), four a wavefront.  64 keys and values at a
// time are staged in LDS as float32 for the whole workgroup; a lane owns one key of the 64 for the
// scores of its wavefront's four rows, then one value channel (and the ones 64 further on) for the
// weighted sum.  Everything is float32; the softmax is the running one (maximum, sum, rescaled sum).
#include "common.h"

#include <algorithm>
#include <cmath>

#define ROWS_PER_WAVE 4
#define WAVES 4
#define ROWS (ROWS_PER_WAVE * WAVES)
#define KEYS 64
#define MAX_VCHUNKS 4          // value channels a lane owns at most: dv <= 256

// Which tiles of KEYS keys a tile of queries (positions first_pos .. last_pos) walks: step v < kept is tile v (the kept
// first keys), step v >= kept the tile at `start + (v - kept) * KEYS`.  Without a window: every tile from key 0.
struct KeyWalk {
    int kept, start, steps;
    __device__ __forceinline__ KeyWalk(int first_pos, int last_pos, int window, int keep_first) {
        kept = 0;
        start = 0;
        if (window > 0) {
            const int lo = max(first_pos - window + 1, 0) / KEYS * KEYS;       // the tile in which the first row's window starts
            const int kept_end = (min(keep_first, last_pos + 1) + KEYS - 1) / KEYS * KEYS;
            if (lo > kept_end) { kept = kept_end / KEYS; start = lo; }
        }
        steps = kept + (last_pos - start) / KEYS + 1;
    }
    __device__ __forceinline__ int first_key(int v) const { return v < kept ? v * KEYS : start + (v - kept) * KEYS; }
};

__device__ __forceinline__ bool key_seen(int key, int pos, int window, int keep_first) {
    return key <= pos && (window <= 0 || pos - key < window || key < keep_first);
}

// keys and values of the step's tokens into their places in the pages
template <typename T>
__global__ void kv_store_kernel(const T* __restrict__ qkv, int row_stride, int k_off, int v_off,
                                const int32_t* __restrict__ slot_mapping, T* __restrict__ kpool, T* __restrict__ vpool,
                                int G, int dk, int dv, int page_size) {
    const int t = blockIdx.x;
    const int slot = slot_mapping[t];
    if (slot < 0) return;
    const int page = slot / page_size, in_page = slot % page_size;
    const T* row = qkv + static_cast<size_t>(t) * row_stride;
    for (int i = threadIdx.x; i < G * dk; i += blockDim.x) {
        const int g = i / dk, c = i % dk;
        kpool[((static_cast<size_t>(page) * G + g) * page_size + in_page) * dk + c] = row[k_off + i];
    }
    for (int i = threadIdx.x; i < G * dv; i += blockDim.x) {
        const int g = i / dv, c = i % dv;
        vpool[((static_cast<size_t>(page) * G + g) * page_size + in_page) * dv + c] = row[v_off + i];
    }
}

// The same for projections that still want their norm and rotation, all of it in float32:
//   q <- rotate(rmsnorm(q) * wq), k <- rotate(rmsnorm(k) * wk)
//   The norms (a null weight: no norm) run over the WHOLE projection of a token, all heads at once, weights [H * dq]
//   and [G * dk]; or, `per_head`, over every head on its own with one weight [dq] (or [k_normed]) shared by the heads.
//   Of a key head only the first `k_normed` channels are normed (whole-projection norms: all of them); the others
//   pass as projected.
//   The rotation (a null freq: none) turns `rot` channels of every head, from channel `rot_at_q` (queries) or
//   `rot_at_k` (keys) on, by the angles position * freq[p], cos and sin times `amplitude`: channel c of them with
//   channel c + rot/2, or, `adjacent`, channel 2p with channel 2p + 1.  The other channels pass as they are.
// proj float32 [T, row_stride] holds q [H * dq] | k [G * dk] | v [G * dv] (`v_from_k`: no v; the values are the keys as
// projected, before their norm, and dv = dk); q goes to q_out [T, H * dq] in the compute
// type, k and v into their page slots.  A token is taken by gridDim.y workgroups, each with its share of the elements
// (and the sums of squares, which every one of them works out): one for steps of many
// tokens; a step of few tokens, where one workgroup a token would walk its row alone, spreads the row.
#define ROT_PAIRS 128          // rotated pairs of a head at most: heads of up to 256 rotated channels
#define NORM_HEADS 1024        // heads of queries and keys together that are normed one by one, at most

struct QkForm {
    int H, G, dq, dk, dv, k_normed, rot, rot_at_q, rot_at_k;
    bool v_from_k, per_head, adjacent;
};

template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_store_kernel(const float* __restrict__ proj, int row_stride, const int32_t* __restrict__ positions,
                          const int32_t* __restrict__ slot_mapping, const float* __restrict__ wq, const float* __restrict__ wk,
                          float eps, const float* __restrict__ freq, float amplitude, T* __restrict__ q_out,
                          T* __restrict__ kpool, T* __restrict__ vpool, int page_size, QkForm f) {
    __shared__ float scratch[8];
    __shared__ float cos_of[ROT_PAIRS], sin_of[ROT_PAIRS];     // the token's angles, worked out once for all heads
    __shared__ float head_r[NORM_HEADS];                       // per_head: 1 / rms of every query head, then of every key head
    const int t = blockIdx.x, tid = threadIdx.x;
    const float* row = proj + static_cast<size_t>(t) * row_stride;
    const int H = f.H, G = f.G, dq = f.dq, dk = f.dk, dv = f.dv, rot = f.rot;
    const int nq = H * dq, nk = G * dk;
    float rq = 1.f, rk = 1.f;
    if (f.per_head) {
        // a head a wavefront at a time: its lanes walk the head's normed channels
        const int lane = tid & (WAVE - 1), wave = tid / WAVE, waves = blockDim.x / WAVE;
        for (int hd = wave; hd < H + G; hd += waves) {
            const bool is_q = hd < H;
            const float* w = is_q ? wq : wk;
            if (!w) continue;                                  // the same for the whole wavefront
            const float* src = is_q ? row + hd * dq : row + nq + (hd - H) * dk;
            const int n = is_q ? dq : f.k_normed;
            float ss = 0.f;
            for (int c = lane; c < n; c += WAVE) ss += src[c] * src[c];
            ss = wave_sum(ss);
            if (lane == 0) head_r[hd] = 1.0f / sqrtf(ss / static_cast<float>(n) + eps);
        }
        __syncthreads();
    } else {
        if (wq) {
            float ss = 0.f;
            for (int i = tid; i < nq; i += blockDim.x) ss += row[i] * row[i];
            rq = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(nq) + eps);
        }
        if (wk) {
            float ss = 0.f;
            for (int i = tid; i < nk; i += blockDim.x) ss += row[nq + i] * row[nq + i];
            rk = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(nk) + eps);
        }
    }
    const float pos = static_cast<float>(positions[t]);
    const int half = rot / 2;
    if (freq) {
        for (int p = tid; p < half; p += blockDim.x) {
            float sn, cs;
            sincosf(pos * freq[p], &sn, &cs);
            cos_of[p] = cs * amplitude;
            sin_of[p] = sn * amplitude;
        }
        __syncthreads();
    }
    const int slot = slot_mapping ? slot_mapping[t] : -1;
    const int page = slot >= 0 ? slot / page_size : 0, in_page = slot >= 0 ? slot % page_size : 0;
    const int slices = gridDim.y, slice = blockIdx.y;
    const int per = ((nq + nk + slices - 1) / slices + 3) / 4 * 4;
    for (int i = slice * per + tid; i < min(nq + nk, (slice + 1) * per); i += blockDim.x) {
        const bool is_q = i < nq;
        const int j = is_q ? i : i - nq;                 // index inside the projection
        const float* src = is_q ? row : row + nq;
        const float* w = is_q ? wq : wk;
        const int size = is_q ? dq : dk;
        const int hd = j / size, c = j - hd * size;
        const int normed = !w ? 0 : (is_q ? size : f.k_normed);       // leading channels of the head that are normed
        const float r = f.per_head ? (w ? head_r[is_q ? hd : H + hd] : 1.f) : (is_q ? rq : rk);
        // the element at channel cc of this head, after its norm
        auto normed_at = [&](int cc) -> float {
            const float x = src[hd * size + cc];
            return cc < normed ? x * r * w[f.per_head ? cc : hd * size + cc] : x;
        };
        float v = normed_at(c);
        const int cr = c - (is_q ? f.rot_at_q : f.rot_at_k);           // index among the rotated channels
        if (freq && cr >= 0 && cr < rot) {
            const bool first = f.adjacent ? !(cr & 1) : cr < half;
            const int partner = f.adjacent ? (cr ^ 1) : (first ? cr + half : cr - half);
            const int p = f.adjacent ? (cr >> 1) : (first ? cr : cr - half);
            const float other = normed_at(c - cr + partner);
            const float cs = cos_of[p], sn = sin_of[p];
            v = first ? v * cs - other * sn : v * cs + other * sn;
        }
        if (is_q) {
            st(q_out + static_cast<size_t>(t) * nq + j, v);
        } else if (slot >= 0) {
            st(kpool + ((static_cast<size_t>(page) * G + hd) * page_size + in_page) * dk + c, v);
        }
    }
    if (slot >= 0) {
        const float* vsrc = f.v_from_k ? row + nq : row + nq + nk;      // the values may be the keys as projected, before their norm
        const int vper = (G * dv + slices - 1) / slices;
        for (int i = slice * vper + tid; i < min(G * dv, (slice + 1) * vper); i += blockDim.x) {
            const int g = i / dv, c = i % dv;
            st(vpool + ((static_cast<size_t>(page) * G + g) * page_size + in_page) * dv + c, vsrc[i]);
        }
    }
}

// `per_head`, `adjacent`, `dq`, `k_normed`, `rot_at_q`, `rot_at_k`: see the kernel.  G may be 0 (queries alone).
NI_EXPORT int ni_qk_norm_rope_store(const void* proj, int row_stride, const void* positions, const void* slot_mapping,
                                    const void* wq, const void* wk, float eps, const void* freq, int rot, float amplitude,
                                    void* q_out, void* kpool, void* vpool, int T, int H, int G, int dq, int dk, int dv, int page_size,
                                    int v_from_k, int per_head, int k_normed, int rot_at_q, int rot_at_k, int adjacent,
                                    int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (H < 0 || G < 0 || dq < 0 || dk < 0 || dv < 0 || (H > 0 && dq < 1) || (G > 0 && dk < 1)) return -1;
    if (rot < 0 || rot % 2 || rot > 2 * ROT_PAIRS || rot_at_q < 0 || rot_at_k < 0) return -1;
    if (freq && ((H > 0 && rot_at_q + rot > dq) || (G > 0 && rot_at_k + rot > dk))) return -1;
    if (row_stride < H * dq + G * dk + (v_from_k ? 0 : G * dv)) return -1;
    if (v_from_k && dv != dk) return -1;
    if (k_normed < 0 || k_normed > dk || (!per_head && wk && k_normed != dk)) return -1;
    if (per_head && H + G > NORM_HEADS) return -1;
    if ((H > 0 && !q_out) || (G > 0 && slot_mapping && (!kpool || (dv > 0 && !vpool)))) return -1;
    const QkForm f{H, G, dq, dk, dv, k_normed, freq ? rot : 0, rot_at_q, rot_at_k, v_from_k != 0, per_head != 0, adjacent != 0};
    // few tokens: a row's elements over several workgroups, one pass of 256 threads each
    const int slices = T >= 64 ? 1 : std::max(1, std::min(16, (H * dq + G * dk + 255) / 256));
    const dim3 grid(T, slices);
    if (dtype == 0)
        qk_norm_rope_store_kernel<float><<<grid, 256, 0, stream>>>((const float*)proj, row_stride, (const int32_t*)positions,
            (const int32_t*)slot_mapping, (const float*)wq, (const float*)wk, eps, (const float*)freq, amplitude,
            (float*)q_out, (float*)kpool, (float*)vpool, page_size, f);
    else
        qk_norm_rope_store_kernel<bf16_t><<<grid, 256, 0, stream>>>((const float*)proj, row_stride, (const int32_t*)positions,
            (const int32_t*)slot_mapping, (const float*)wq, (const float*)wk, eps, (const float*)freq, amplitude,
            (bf16_t*)q_out, (bf16_t*)kpool, (bf16_t*)vpool, page_size, f);
    return NI_LAUNCH_RESULT();
}

// 64 rows of a pool (keys or values of one kv head) from their pages into LDS as float32, row stride `stride`.
// With `pieces` (rows of whole 16-byte pieces, 16-byte aligned) a thread asks for four pieces before it stores
// the first: the loads of a tile are then in flight together instead of one round trip after the other.
template <typename T>
__device__ __forceinline__ void stage_rows(const T* __restrict__ pool, float* __restrict__ dst, int stride, int size,
                                           const int32_t* __restrict__ table, int page_size, int G, int g, int k0,
                                           int k_last, bool pieces) {
    constexpr int VEC = 16 / sizeof(T);
    const int tid = threadIdx.x, threads = blockDim.x;
    if (pieces) {
        const int per_row = size / VEC, total = KEYS * per_row;
        for (int base = 0; base < total; base += 4 * threads) {
            RawRow<T, VEC> raw[4];
            bool have[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * threads + tid;
                have[u] = false;
                if (idx < total) {
                    const int j = idx / per_row, pc = idx % per_row, key = k0 + j;
                    if (key <= k_last) {
                        const int page = table[key / page_size];
                        if (page >= 0) {
                            raw[u].load(pool + ((static_cast<size_t>(page) * G + g) * page_size + key % page_size) * size + pc * VEC);
                            have[u] = true;
                        }
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int idx = base + u * threads + tid;
                if (idx < total) {
                    float* d = dst + (idx / per_row) * stride + (idx % per_row) * VEC;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) d[e] = have[u] ? raw[u].get(e) : 0.f;
                }
            }
        }
        return;
    }
    for (int i = tid; i < KEYS * size; i += threads) {
        const int j = i / size, c = i % size, key = k0 + j;
        float v = 0.f;
        if (key <= k_last) {
            const int page = table[key / page_size];
            if (page >= 0) v = ld(pool + ((static_cast<size_t>(page) * G + g) * page_size + key % page_size) * size + c);
        }
        dst[j * stride + c] = v;
    }
}

// The same in two halves, for tiles whose rows are at most four 16-byte pieces a thread: what stage_rows would
// load, asked for and kept in registers, and its way into LDS afterwards.  Keys and values asked for one after the
// other and stored after both are on their way together: one round trip to memory a tile instead of two.
template <typename T> struct StagedRows {
    RawRow<T, 16 / sizeof(T)> raw[4];
    bool have[4];
};

template <typename T>
__device__ __forceinline__ void stage_ask(const T* __restrict__ pool, StagedRows<T>& x, int size, const int32_t* __restrict__ table,
                                          int page_size, int G, int g, int k0, int k_last) {
    constexpr int VEC = 16 / sizeof(T);
    const int tid = threadIdx.x, threads = blockDim.x;
    const int per_row = size / VEC, total = KEYS * per_row;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int idx = u * threads + tid;
        x.have[u] = false;
        if (idx < total) {
            const int j = idx / per_row, pc = idx % per_row, key = k0 + j;
            if (key <= k_last) {
                const int page = table[key / page_size];
                if (page >= 0) {
                    x.raw[u].load(pool + ((static_cast<size_t>(page) * G + g) * page_size + key % page_size) * size + pc * VEC);
                    x.have[u] = true;
                }
            }
        }
    }
}

template <typename T>
__device__ __forceinline__ void stage_put(const StagedRows<T>& x, float* __restrict__ dst, int stride, int size) {
    constexpr int VEC = 16 / sizeof(T);
    const int tid = threadIdx.x, threads = blockDim.x;
    const int per_row = size / VEC, total = KEYS * per_row;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int idx = u * threads + tid;
        if (idx < total) {
            float* d = dst + (idx / per_row) * stride + (idx % per_row) * VEC;
#pragma unroll
            for (int e = 0; e < VEC; ++e) d[e] = x.have[u] ? x.raw[u].get(e) : 0.f;
        }
    }
}

// keys and values of a tile into LDS: together where both fit four pieces a thread, else one after the other
template <typename T>
__device__ __forceinline__ void stage_tile(const T* __restrict__ kpool, const T* __restrict__ vpool, float* __restrict__ Ks, int dkp,
                                           int dk, float* __restrict__ Vs, int dvp, int dv, const int32_t* __restrict__ table,
                                           int page_size, int G, int g, int k0, int k_last, bool k_pieces, bool v_pieces) {
    constexpr int VEC = 16 / sizeof(T);
    const int room = 4 * blockDim.x;
    if (k_pieces && v_pieces && KEYS * (dk / VEC) <= room && KEYS * (dv / VEC) <= room) {
        StagedRows<T> k, v;
        stage_ask<T>(kpool, k, dk, table, page_size, G, g, k0, k_last);
        stage_ask<T>(vpool, v, dv, table, page_size, G, g, k0, k_last);
        stage_put<T>(k, Ks, dkp, dk);
        stage_put<T>(v, Vs, dvp, dv);
        return;
    }
    stage_rows<T>(kpool, Ks, dkp, dk, table, page_size, G, g, k0, k_last, k_pieces);
    stage_rows<T>(vpool, Vs, dvp, dv, table, page_size, G, g, k0, k_last, v_pieces);
}

template <typename T>
__global__ void __launch_bounds__(WAVES * WAVE)
bias_attention_kernel(const T* __restrict__ qkv, int row_stride, const T* __restrict__ kpool, const T* __restrict__ vpool,
                      const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
                      const int32_t* __restrict__ positions, const float* __restrict__ bias, int distances, T* __restrict__ out, int H, int G, int dk, int dv,
                      int page_size, float scale, float temp_coef, int temp_every, int heads_per_chunk, int n_runs,
                      float* __restrict__ partial, bool k_pieces, bool v_pieces, int dkp, int window, int keep_first,
                      float out_scale, const float* __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    // a lane reads its key's row: the stride is the row plus four floats where rows are whole 16-byte pieces (read
    // as such), plus one otherwise; both spread the lanes over the banks
    float* Qs = lds;                              // [ROWS][dk]
    float* Ks = Qs + ROWS * dk;                   // [KEYS][dkp]
    float* Vs = Ks + KEYS * dkp;                  // [KEYS][dv]
    float* Ps = Vs + KEYS * dv;                   // [WAVES][ROWS_PER_WAVE][KEYS]
    // with n_runs > 1 the keys of a tile are cut into runs, one workgroup each, whose (maximum, sum, weighted
    // sum) a second kernel merges: a single token over thousands of keys then fills the chip
    const int tile = blockIdx.x / n_runs, run = blockIdx.x % n_runs, g = blockIdx.y, chunk = blockIdx.z;
    // the first position is read from the step's positions, not from the tile: a recorded decode step is replayed
    // with new positions and the tiles it was recorded with
    const int seq = tiles[4 * tile], first_row = tiles[4 * tile + 1], n_tok = tiles[4 * tile + 2];
    const int first_pos = positions[first_row];
    const int group = H / G;
    const int heads_here = std::min(heads_per_chunk, group - chunk * heads_per_chunk);
    const int head0 = g * group + chunk * heads_per_chunk;
    const int n_rows = n_tok * heads_here;        // row r = token r / heads_here, head r % heads_here
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;

    for (int i = tid; i < ROWS * dk; i += blockDim.x) {
        const int r = i / dk, c = i % dk;
        float v = 0.f;
        if (r < n_rows)
            v = ld(qkv + static_cast<size_t>(first_row + r / heads_here) * row_stride + (head0 + r % heads_here) * dk + c);
        Qs[i] = v;
    }
    float m[ROWS_PER_WAVE], l[ROWS_PER_WAVE], acc[ROWS_PER_WAVE][MAX_VCHUNKS], factor[ROWS_PER_WAVE];
    int pos[ROWS_PER_WAVE], head[ROWS_PER_WAVE];
    bool valid[ROWS_PER_WAVE];
#pragma unroll
    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
        const int r = wave * ROWS_PER_WAVE + rr;
        valid[rr] = r < n_rows;
        pos[rr] = first_pos + (valid[rr] ? r / heads_here : 0);
        head[rr] = head0 + (valid[rr] ? r % heads_here : 0);
        const int steps = temp_every > 0 ? (pos[rr] + 1) / temp_every : 0;
        factor[rr] = scale * (1.0f + temp_coef * logf(static_cast<float>(steps) + 1.0f));
        m[rr] = -INFINITY;
        l[rr] = 0.f;
#pragma unroll
        for (int cc = 0; cc < MAX_VCHUNKS; ++cc) acc[rr][cc] = 0.f;
    }
    const int last_pos = first_pos + n_tok - 1;
    const KeyWalk walk(first_pos, last_pos, window, keep_first);
    const int per_run = (walk.steps + n_runs - 1) / n_runs;                        // tiles of 64 keys a run
    const int v_end = std::min(walk.steps, (run + 1) * per_run);
    const int k_last = last_pos;
    const int32_t* table = block_table + static_cast<size_t>(seq) * table_width;
    for (int v = run * per_run; v < v_end; ++v) {
        const int k0 = walk.first_key(v);
        __syncthreads();                          // the tile before this one has been used by everyone
        stage_tile<T>(kpool, vpool, Ks, dkp, dk, Vs, dv, dv, table, page_size, G, g, k0, k_last, k_pieces, v_pieces);
        __syncthreads();
        // scores of this lane's key for the wavefront's rows
        float s[ROWS_PER_WAVE];
#pragma unroll
        for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) s[rr] = 0.f;
        const float* krow = Ks + lane * dkp;
        const float* qrow = Qs + wave * ROWS_PER_WAVE * dk;
        if (dkp == dk + 4) {
            for (int c = 0; c < dk; c += 4) {
                const float4 kv = *reinterpret_cast<const float4*>(krow + c);
#pragma unroll
                for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
                    const float4 q = *reinterpret_cast<const float4*>(qrow + rr * dk + c);
                    s[rr] += q.x * kv.x + q.y * kv.y + q.z * kv.z + q.w * kv.w;
                }
            }
        } else {
            for (int c = 0; c < dk; ++c) {
                const float kv = krow[c];
#pragma unroll
                for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) s[rr] += qrow[rr * dk + c] * kv;
            }
        }
        const int key = k0 + lane;
        float* prow = Ps + wave * ROWS_PER_WAVE * KEYS;
        float alpha[ROWS_PER_WAVE];
#pragma unroll
        for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
            alpha[rr] = 1.f;
            if (!valid[rr]) { prow[rr * KEYS + lane] = 0.f; continue; }          // the same for the whole wavefront
            if (k0 > pos[rr]) { prow[rr * KEYS + lane] = 0.f; continue; }        // the same for the whole wavefront
            const bool seen = key_seen(key, pos[rr], window, keep_first);
            float sc = -INFINITY;
            if (seen) {
                const int back = std::min(pos[rr] - key, distances - 1);
                sc = s[rr] * factor[rr] + (bias ? bias[static_cast<size_t>(back) * H + head[rr]] : 0.f);
            }
            const float m_new = fmaxf(m[rr], wave_max(sc));
            if (m_new == -INFINITY) { prow[rr * KEYS + lane] = 0.f; continue; }   // no key of this row so far (a window that starts later)
            alpha[rr] = expf(m[rr] - m_new);                      // 0 at the row's first keys
            const float p = seen ? expf(sc - m_new) : 0.f;
            l[rr] = l[rr] * alpha[rr] + wave_sum(p);
            m[rr] = m_new;
            prow[rr * KEYS + lane] = p;
        }
        // a wavefront reads only what it wrote itself: no barrier of the workgroup is needed here
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int cc = 0; cc < MAX_VCHUNKS; ++cc) {
            const int c = lane + cc * WAVE;
            if (c < dv) {
                float add[ROWS_PER_WAVE];
#pragma unroll
                for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) add[rr] = 0.f;
                for (int j = 0; j < KEYS; j += 4) {
                    const float v0 = Vs[j * dv + c], v1 = Vs[(j + 1) * dv + c], v2 = Vs[(j + 2) * dv + c], v3 = Vs[(j + 3) * dv + c];
#pragma unroll
                    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
                        const float4 p = *reinterpret_cast<const float4*>(prow + rr * KEYS + j);
                        add[rr] += p.x * v0 + p.y * v1 + p.z * v2 + p.w * v3;
                    }
                }
#pragma unroll
                for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) acc[rr][cc] = acc[rr][cc] * alpha[rr] + add[rr];
            }
        }
    }
#pragma unroll
    for (int rr = 0; rr < ROWS_PER_WAVE; ++rr) {
        if (!valid[rr]) continue;
        const int r = wave * ROWS_PER_WAVE + rr;
        if (partial) {
            float* prow = partial + ((static_cast<size_t>(first_row + r / heads_here) * H + head[rr]) * n_runs + run) * (dv + 2);
            if (lane == 0) { prow[0] = m[rr]; prow[1] = l[rr]; }
#pragma unroll
            for (int cc = 0; cc < MAX_VCHUNKS; ++cc) {
                const int c = lane + cc * WAVE;
                if (c < dv) prow[2 + c] = acc[rr][cc];
            }
            continue;
        }
        T* orow = out + static_cast<size_t>(first_row + r / heads_here) * (H * dv) + head[rr] * dv;
        float inv = out_scale / l[rr];
        if (sink) {             // one more term in the denominator: with M = max(m, sink), l e^(m - M) + e^(sink - M)
            const float sk = sink[head[rr]], M = fmaxf(m[rr], sk), w = expf(m[rr] - M);
            inv = out_scale * w / (l[rr] * w + expf(sk - M));
        }
#pragma unroll
        for (int cc = 0; cc < MAX_VCHUNKS; ++cc) {
            const int c = lane + cc * WAVE;
            if (c < dv) st(orow + c, acc[rr][cc] * inv);
        }
    }
}

// ------------------------------------------------------------------ prompt portions on the matrix cores, in float32
// The same attention for tiles of up to 64 rows of (token, head), sixteen a wavefront, with both products on
// v_mfma_f32_16x16x4_f32 (true 32-bit products and sums; keys, values and queries are widened to float32 when they
// are staged).  Key and value sizes are multiples of 16.
//
//   S^T[key, row]  = K[key, :] . Q[row, :]    K rows as the first operand, Q rows as the second.  The k index of
//                    an MFMA is only a label: lane group kg (lane / 16) of step t takes channel kg dk/4 + t, so
//                    a lane reads dk/4 consecutive floats of its key and of its row.  A lane ends up with the
//                    scores of ONE row (lane % 16) for keys 16 j + 4 kg + r: bias, temperature and the running
//                    softmax are per lane, the row's maximum and sum cross the four lane groups only.
//   O^T[dim, row] += V^T[dim, key] . P^T[key, row]   the weight of key 16 j + 4 kg + r is register (j, r) of the
//                    lane, which is where the second operand of the MFMA over keys {16 j + 4 kg + r} wants it:
//                    the weights never leave the registers.  The lane holds dims 16 db + 4 kg + r of its row.
#define MROWS 64
typedef float floatx4_t __attribute__((ext_vector_type(4)));

// floats of the first region of the kernel's staging memory: the queries [MROWS][dk + 4], whose place the tiles of values
// [KEYS][dv + 4] take once the queries are in registers (no tile of values where keys and values are one pool)
__host__ __device__ __forceinline__ size_t mfma_first_floats(int dk, int dv, bool one_pool) {
    const size_t q = static_cast<size_t>(MROWS) * (dk + 4), v = one_pool ? 0 : static_cast<size_t>(KEYS) * (dv + 4);
    return q > v ? q : v;
}

__device__ __forceinline__ float groups4(float x, bool take_max) {
    // over the four lanes that hold one row (lanes r, r + 16, r + 32, r + 48): maximum or sum
    const auto a = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float u = __uint_as_float(a[0]), v = __uint_as_float(a[1]);
    x = take_max ? fmaxf(u, v) : u + v;
    const auto b = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    const float s = __uint_as_float(b[0]), t = __uint_as_float(b[1]);
    return take_max ? fmaxf(s, t) : s + t;
}

// QS: 16-byte pieces of a lane's quarter of a query row at most (dk <= 64 QS); DVB: blocks of 16 value channels at most
// (dv <= 16 DVB).  Both size arrays of registers, so the kernel is compiled for a few pairs of them.
template <typename T, int QS, int DVB>
__global__ void __launch_bounds__(WAVES * WAVE)
bias_attention_mfma_kernel(const T* __restrict__ qkv, int row_stride, const T* __restrict__ kpool, const T* __restrict__ vpool,
                           const int32_t* __restrict__ block_table, int table_width, const int32_t* __restrict__ tiles,
                           const int32_t* __restrict__ positions, const float* __restrict__ bias, int distances,
                           T* __restrict__ out, int H, int G, int dk, int dv, int page_size, float scale, float temp_coef,
                           int temp_every, int heads_per_chunk, bool k_pieces, bool v_pieces, int window, int keep_first,
                           float out_scale, const float* __restrict__ sink) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int dkp = dk + 4, dvp = dv + 4;         // strides that spread the sixteen rows of a read over the banks
    // keys and values that are one pool (dv = dk) are staged once: the values are read from the keys' tile
    const bool one_pool = static_cast<const void*>(kpool) == static_cast<const void*>(vpool) && dk == dv;
    // the queries are staged once and then live in registers, a lane's quarter of its row; the tiles of values take
    // their place in LDS
    float* Qs = lds;                              // [MROWS][dkp], later [KEYS][dvp]
    float* Ks = lds + mfma_first_floats(dk, dv, one_pool);      // [KEYS][dkp]
    float* Vs = one_pool ? Ks : lds;
    const int tile = blockIdx.x, g = blockIdx.y, chunk = blockIdx.z;
    const int seq = tiles[4 * tile], first_row = tiles[4 * tile + 1], n_tok = tiles[4 * tile + 2];
    const int first_pos = positions[first_row];
    const int group = H / G;
    const int heads_here = std::min(heads_per_chunk, group - chunk * heads_per_chunk);
    const int head0 = g * group + chunk * heads_per_chunk;
    const int n_rows = n_tok * heads_here;        // row r = token r / heads_here, head r % heads_here
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int i = lane & 15, kg = lane >> 4;

    for (int e = tid; e < MROWS * dk; e += blockDim.x) {
        const int r = e / dk, c = e % dk;
        float v = 0.f;
        if (r < n_rows)
            v = ld(qkv + static_cast<size_t>(first_row + r / heads_here) * row_stride + (head0 + r % heads_here) * dk + c);
        Qs[r * dkp + c] = v;
    }
    const int row = wave * 16 + i;
    const bool valid = row < n_rows;
    const int pos = first_pos + (valid ? row / heads_here : 0);
    const int head = head0 + (valid ? row % heads_here : 0);
    const int steps = temp_every > 0 ? (pos + 1) / temp_every : 0;
    const float factor = scale * (1.0f + temp_coef * logf(static_cast<float>(steps) + 1.0f));
    // the last position any row of this wavefront has (the same for all its lanes)
    const int wave_rows = std::min(16, n_rows - wave * 16);
    const int wave_last = wave_rows > 0 ? first_pos + (wave * 16 + wave_rows - 1) / heads_here : -1;
    float m = -INFINITY, l = 0.f;
    floatx4_t acc[DVB];                           // dv / 16 blocks of [4 dims] of the lane's row
#pragma unroll
    for (int db = 0; db < DVB; ++db) acc[db] = floatx4_t{0.f, 0.f, 0.f, 0.f};
    const int dvb = dv / 16, qsteps = dk / 16;    // value blocks; 16-byte reads of a lane's quarter of a row
    const int last_pos = first_pos + n_tok - 1;
    const int32_t* table = block_table + static_cast<size_t>(seq) * table_width;
    const float* qrow = Qs + row * dkp + kg * (dk / 4);
    __syncthreads();                              // the queries are all there
    float4 qreg[QS];
#pragma unroll
    for (int t4 = 0; t4 < QS; ++t4)
        qreg[t4] = t4 < qsteps ? *reinterpret_cast<const float4*>(qrow + 4 * t4) : make_float4(0.f, 0.f, 0.f, 0.f);
    const KeyWalk walk(first_pos, last_pos, window, keep_first);
    for (int v = 0; v < walk.steps; ++v) {
        const int k0 = walk.first_key(v);
        __syncthreads();                          // the tile before this one has been used by everyone
        // one after the other: both in registers at once would cost this kernel its second wavefront a SIMD
        stage_rows<T>(kpool, Ks, dkp, dk, table, page_size, G, g, k0, last_pos, k_pieces);
        if (!one_pool) stage_rows<T>(vpool, Vs, dvp, dv, table, page_size, G, g, k0, last_pos, v_pieces);
        __syncthreads();
        if (k0 > wave_last) continue;             // nothing here for this wavefront's rows (it still stages and waits)
        floatx4_t sc[KEYS / 16];
#pragma unroll
        for (int j = 0; j < KEYS / 16; ++j) sc[j] = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t4 = 0; t4 < QS; ++t4) {
            if (t4 < qsteps) {
                const float4 qv = qreg[t4];
#pragma unroll
                for (int j = 0; j < KEYS / 16; ++j) {
                    const float4 kv = *reinterpret_cast<const float4*>(Ks + (16 * j + i) * dkp + kg * (dk / 4) + 4 * t4);
                    sc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv.x, qv.x, sc[j], 0, 0, 0);
                    sc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv.y, qv.y, sc[j], 0, 0, 0);
                    sc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv.z, qv.z, sc[j], 0, 0, 0);
                    sc[j] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv.w, qv.w, sc[j], 0, 0, 0);
                }
            }
        }
        float top = -INFINITY;
#pragma unroll
        for (int j = 0; j < KEYS / 16; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = k0 + 16 * j + 4 * kg + r;
                float v = -INFINITY;
                if (valid && key_seen(key, pos, window, keep_first)) {
                    const int back = std::min(pos - key, distances - 1);
                    v = sc[j][r] * factor + (bias ? bias[static_cast<size_t>(back) * H + head] : 0.f);
                }
                sc[j][r] = v;
                top = fmaxf(top, v);
            }
        top = groups4(top, true);
        const float m_new = fmaxf(m, top);
        const bool any = m_new > -INFINITY;       // a row that is no row, or whose keys all lie ahead, sees nothing
        const float alpha = any ? expf(m - m_new) : 1.f;          // 0 at the row's first keys
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < KEYS / 16; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float p = any ? expf(sc[j][r] - m_new) : 0.f;           // e^-inf = 0 for a key that is not seen
                sc[j][r] = p;
                sum += p;
            }
        l = l * alpha + groups4(sum, false);
        m = m_new;
#pragma unroll
        for (int db = 0; db < DVB; ++db) {
            if (db < dvb) {
                floatx4_t a = acc[db] * alpha;
#pragma unroll
                for (int j = 0; j < KEYS / 16; ++j)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        a = __builtin_amdgcn_mfma_f32_16x16x4f32(Vs[(16 * j + 4 * kg + r) * dvp + 16 * db + i], sc[j][r], a, 0, 0, 0);
                acc[db] = a;
            }
        }
    }
    if (!valid) return;
    T* orow = out + static_cast<size_t>(first_row + row / heads_here) * (H * dv) + head * dv + 4 * kg;
    float inv = out_scale / l;
    if (sink) {                 // one more term in the denominator: with M = max(m, sink), l e^(m - M) + e^(sink - M)
        const float sk = sink[head], M = fmaxf(m, sk), w = expf(m - M);
        inv = out_scale * w / (l * w + expf(sk - M));
    }
#pragma unroll
    for (int db = 0; db < DVB; ++db) {
        if (db < dvb) {
#pragma unroll
            for (int r = 0; r < 4; ++r) st(orow + 16 * db + r, acc[db][r] * inv);
        }
    }
}

// out[row, :] = sum_r acc_r e^(m_r - M) / (sum_r l_r e^(m_r - M) + e^(sink - M)) over the runs of a row (an empty run
// has l = 0; no sink: no such term; M is the maximum over the runs and the sink).
// The weights e^(m_r - M) go through LDS, and the sums over the runs then read nothing that depends on an earlier read.
// One workgroup a row, of as many wavefronts as the row has runs of 64 value channels (up to four); every wavefront works
// the runs' weights out for itself (lane r takes run r's maximum and sum, n_runs <= 64) and sums its own channels.
template <typename T>
__global__ void __launch_bounds__(MAX_VCHUNKS * WAVE) merge_runs_kernel(const float* __restrict__ partial, T* __restrict__ out, int n_runs,
                                                                        int dv, float out_scale, const float* __restrict__ sink, int H) {
    __shared__ float weight[MAX_VCHUNKS][WAVE];
    const size_t row = blockIdx.x;
    const float* p = partial + row * n_runs * (dv + 2);
    const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
    float m = -INFINITY, l = 0.f;
    if (lane < n_runs) {
        m = p[lane * (dv + 2)];
        l = p[lane * (dv + 2) + 1];
    }
    if (!(l > 0.f)) m = -INFINITY;
    float M = wave_max(m);
    const float sk = sink ? sink[row % H] : -INFINITY;        // rows are (token, head); the sink counts once, here
    M = fmaxf(M, sk);
    const float w = l > 0.f ? expf(m - M) : 0.f;
    const float L = wave_sum(l * w) + (sink ? expf(sk - M) : 0.f);
    weight[wave][lane] = w;
    __builtin_amdgcn_wave_barrier();          // a wavefront reads only the weights it wrote itself
    for (int c = wave * WAVE + lane; c < dv; c += blockDim.x) {
        float a = 0.f;
        for (int r = 0; r < n_runs; ++r) {
            const float wr = weight[wave][r];
            if (wr > 0.f) a += p[r * (dv + 2) + 2 + c] * wr;
        }
        st(out + row * dv + c, a * out_scale / L);
    }
}

NI_EXPORT int ni_kv_store(const void* qkv, int row_stride, int k_off, int v_off, const void* slot_mapping, void* kpool,
                          void* vpool, int T, int G, int dk, int dv, int page_size, int dtype, hipStream_t stream) {
    if (T <= 0) return 0;
    if (dtype == 0)
        kv_store_kernel<float><<<T, 256, 0, stream>>>((const float*)qkv, row_stride, k_off, v_off, (const int32_t*)slot_mapping,
                                                      (float*)kpool, (float*)vpool, G, dk, dv, page_size);
    else
        kv_store_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)qkv, row_stride, k_off, v_off, (const int32_t*)slot_mapping,
                                                       (bf16_t*)kpool, (bf16_t*)vpool, G, dk, dv, page_size);
    return NI_LAUNCH_RESULT();
}

NI_EXPORT int ni_bias_attention_rows() { return ROWS; }

NI_EXPORT int ni_bias_attention(const void* qkv, int row_stride, const void* kpool, const void* vpool, const void* block_table,
                                int table_width, const void* tiles, int n_tiles, const void* positions, const void* bias, int distances, void* out,
                                int H, int G, int dk, int dv, int page_size, float scale, float temp_coef, int temp_every,
                                int heads_per_chunk, int n_runs, void* partial, int n_rows, int waves, int window, int keep_first,
                                float out_scale, const void* sink, int dtype, hipStream_t stream) {
    if (n_tiles <= 0) return 0;
    if (window < 0 || keep_first < 0) return -1;
    if (dv > MAX_VCHUNKS * WAVE || H % G || heads_per_chunk < 1 || heads_per_chunk > ROWS) return -1;
    const int group = H / G;
    const int dkp = dk % 4 == 0 ? dk + 4 : dk + 1;
    const size_t lds = (static_cast<size_t>(ROWS) * dk + static_cast<size_t>(KEYS) * dkp + static_cast<size_t>(KEYS) * dv +
                        WAVES * ROWS_PER_WAVE * KEYS) * sizeof(float);
    if (lds > 160 * 1024) return -2;
    if (n_runs < 1 || (n_runs > 1 && !partial) || waves < 1 || waves > WAVES) return -1;
    const int vec = dtype == 0 ? 4 : 8;
    const bool k_pieces = dk % vec == 0 && reinterpret_cast<uintptr_t>(kpool) % 16 == 0;
    const bool v_pieces = dv % vec == 0 && reinterpret_cast<uintptr_t>(vpool) % 16 == 0;
    if (n_runs == 1) partial = nullptr;
    dim3 grid(n_tiles * n_runs, G, (group + heads_per_chunk - 1) / heads_per_chunk);
    hipError_t err = hipSuccess;
    if (dtype == 0) {
        static size_t allowed = 48 * 1024;
        if (lds > allowed && (allowed = lds))
            err = hipFuncSetAttribute((const void*)bias_attention_kernel<float>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return (int)err;
        bias_attention_kernel<float><<<grid, waves * WAVE, lds, stream>>>(
            (const float*)qkv, row_stride, (const float*)kpool, (const float*)vpool, (const int32_t*)block_table, table_width,
            (const int32_t*)tiles, (const int32_t*)positions, (const float*)bias, distances, (float*)out, H, G, dk, dv, page_size, scale, temp_coef,
            temp_every, heads_per_chunk, n_runs, (float*)partial, k_pieces, v_pieces, dkp, window, keep_first, out_scale,
            (const float*)sink);
        if (partial) merge_runs_kernel<float><<<n_rows * H, std::min(MAX_VCHUNKS, (dv + WAVE - 1) / WAVE) * WAVE, 0, stream>>>((const float*)partial, (float*)out, n_runs, dv, out_scale,
                                                                             (const float*)sink, H);
    } else {
        static size_t allowed = 48 * 1024;
        if (lds > allowed && (allowed = lds))
            err = hipFuncSetAttribute((const void*)bias_attention_kernel<bf16_t>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return (int)err;
        bias_attention_kernel<bf16_t><<<grid, waves * WAVE, lds, stream>>>(
            (const bf16_t*)qkv, row_stride, (const bf16_t*)kpool, (const bf16_t*)vpool, (const int32_t*)block_table, table_width,
            (const int32_t*)tiles, (const int32_t*)positions, (const float*)bias, distances, (bf16_t*)out, H, G, dk, dv, page_size, scale, temp_coef,
            temp_every, heads_per_chunk, n_runs, (float*)partial, k_pieces, v_pieces, dkp, window, keep_first, out_scale,
            (const float*)sink);
        if (partial) merge_runs_kernel<bf16_t><<<n_rows * H, std::min(MAX_VCHUNKS, (dv + WAVE - 1) / WAVE) * WAVE, 0, stream>>>((const float*)partial, (bf16_t*)out, n_runs, dv, out_scale,
                                                                              (const float*)sink, H);
    }
    return NI_LAUNCH_RESULT();
}

// staging memory of the matrix-core kernel: the queries (then the tiles of values) and a tile of keys
static size_t mfma_lds_bytes(int dk, int dv, bool one_pool) {
    return (mfma_first_floats(dk, dv, one_pool) + static_cast<size_t>(KEYS) * (dk + 4)) * sizeof(float);
}

// rows of (token, head) of a tile of the matrix-core kernel; 0 where it does not take these sizes.  `one_pool`: keys
// and values are the same pool (dv = dk)
NI_EXPORT int ni_bias_attention_mfma_rows(int dk, int dv, int one_pool) {
    if (dk % 16 || dv % 16 || dk < 16 || dv < 16 || dv > MAX_VCHUNKS * WAVE || (one_pool && dk != dv)) return 0;
    return mfma_lds_bytes(dk, dv, one_pool != 0) <= 160 * 1024 ? MROWS : 0;
}

struct MfmaArgs {
    const void *qkv; int row_stride; const void *kpool, *vpool, *block_table; int table_width; const void *tiles, *positions, *bias;
    int distances; void* out; int H, G, dk, dv, page_size; float scale, temp_coef; int temp_every, heads_per_chunk;
    bool k_pieces, v_pieces; int window, keep_first; float out_scale; const void* sink;
};

template <typename T, int QS, int DVB>
static hipError_t launch_mfma(const MfmaArgs& a, dim3 grid, size_t lds, hipStream_t stream) {
    static size_t allowed = 48 * 1024;            // of this instance of the kernel
    if (lds > allowed) {
        const hipError_t err = hipFuncSetAttribute((const void*)bias_attention_mfma_kernel<T, QS, DVB>,
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
        allowed = lds;
    }
    bias_attention_mfma_kernel<T, QS, DVB><<<grid, WAVES * WAVE, lds, stream>>>(
        (const T*)a.qkv, a.row_stride, (const T*)a.kpool, (const T*)a.vpool, (const int32_t*)a.block_table, a.table_width,
        (const int32_t*)a.tiles, (const int32_t*)a.positions, (const float*)a.bias, a.distances, (T*)a.out, a.H, a.G, a.dk, a.dv,
        a.page_size, a.scale, a.temp_coef, a.temp_every, a.heads_per_chunk, a.k_pieces, a.v_pieces, a.window, a.keep_first,
        a.out_scale, (const float*)a.sink);
    return hipSuccess;
}

// tiles of up to 64 rows (tokens * heads of a chunk), no runs: for steps with portions of prompts
NI_EXPORT int ni_bias_attention_mfma(const void* qkv, int row_stride, const void* kpool, const void* vpool, const void* block_table,
                                     int table_width, const void* tiles, int n_tiles, const void* positions, const void* bias,
                                     int distances, void* out, int H, int G, int dk, int dv, int page_size, float scale,
                                     float temp_coef, int temp_every, int heads_per_chunk, int window, int keep_first,
                                     float out_scale, const void* sink, int dtype, hipStream_t stream) {
    if (n_tiles <= 0) return 0;
    if (window < 0 || keep_first < 0) return -1;
    const bool one_pool = kpool == vpool && dk == dv;
    if (!ni_bias_attention_mfma_rows(dk, dv, one_pool) || H % G || heads_per_chunk < 1 || heads_per_chunk > MROWS) return -1;
    const int group = H / G;
    const size_t lds = mfma_lds_bytes(dk, dv, one_pool);
    const int vec = dtype == 0 ? 4 : 8;
    const bool k_pieces = dk % vec == 0 && reinterpret_cast<uintptr_t>(kpool) % 16 == 0;
    const bool v_pieces = dv % vec == 0 && reinterpret_cast<uintptr_t>(vpool) % 16 == 0;
    dim3 grid(n_tiles, G, (group + heads_per_chunk - 1) / heads_per_chunk);
    const MfmaArgs args{qkv, row_stride, kpool, vpool, block_table, table_width, tiles, positions, bias, distances, out, H, G, dk, dv,
                        page_size, scale, temp_coef, temp_every, heads_per_chunk, k_pieces, v_pieces, window, keep_first, out_scale, sink};
    hipError_t err;
    // the smallest arrays of registers that hold these sizes
    if (dk <= 64 && dv <= 64) err = dtype == 0 ? launch_mfma<float, 4, 4>(args, grid, lds, stream) : launch_mfma<bf16_t, 4, 4>(args, grid, lds, stream);
    else if (dk <= 128 && dv <= 64) err = dtype == 0 ? launch_mfma<float, 8, 4>(args, grid, lds, stream) : launch_mfma<bf16_t, 8, 4>(args, grid, lds, stream);
    else if (dk <= 128) err = dtype == 0 ? launch_mfma<float, 8, 16>(args, grid, lds, stream) : launch_mfma<bf16_t, 8, 16>(args, grid, lds, stream);
    else err = dtype == 0 ? launch_mfma<float, 16, 16>(args, grid, lds, stream) : launch_mfma<bf16_t, 16, 16>(args, grid, lds, stream);
    if (err != hipSuccess) return (int)err;
    return NI_LAUNCH_RESULT();
}
