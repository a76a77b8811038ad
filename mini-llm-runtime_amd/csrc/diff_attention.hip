// Differential attention over the paged cache.
//
// A query head holds two maps: two softmax attentions with queries and keys of their own (head_dim channels
// each, laid out [map 1 | map 2] within a head) over the SAME values (value_dim channels).  The head's output
// is o = a1 - lam * a2, divided by its root mean square over the value channels (eps inside the root), times
// out_scale, times an activation of the head's gate.  Scores: (q . k) * scale * temp(p), the query's factor
// temp(p) = 1 + coef * ln(floor((p + 1) / every) + 1) growing with its position p; then, with a cap,
// score <- cap * tanh(score / cap); position p sees the keys 0 .. p.  All of this is 32-bit.
//
// Cache of one layer: keys pages[num_pages][kv_heads][page_size][2 * head_dim], values
// pages[num_pages][kv_heads][page_size][value_dim].  Query head h reads kv head h / (q_heads / kv_heads).
//
// `diff_attention_partial_kernel`: one wavefront per (token, head and map, key range).  Key ranges are
// [s * split_keys, (s + 1) * split_keys) in absolute positions and tiles of 64 keys start at multiples of 64, so
// the order of a token's sums follows from its own position alone, never from the batch around it or from how
// its request was cut into steps.  It leaves (max, sum, weighted values) per range;
// `diff_attention_combine_kernel` merges the ranges in ascending order, takes the difference of the maps, norms
// and gates.
#include "common.h"

#define TILE_KEYS 64
#define DIM_CHUNK 64
#define MAX_V_REGS 4            // value_dim <= 64 * MAX_V_REGS
#define COMBINE_MAX_SPLITS 1024

struct DiffArgs {
    const elem_t* q; long q_stride;            // q[m * q_stride + (head * 2 + map) * head_dim + d]
    const elem_t* k_pages; const elem_t* v_pages;
    const int32_t* block_table; const int32_t* slots; const int32_t* positions;
    const elem_t* gate; long gate_stride;      // gate[m * gate_stride + head * value_dim + c], or null
    elem_t* out;                               // [rows, q_heads * value_dim]
    float* partial;                            // [rows, q_heads * 2, max_splits, value_dim + 2]
    int max_blocks, q_heads, kv_heads, head_dim, value_dim, page_size, split_keys, max_splits;
    float scale, softcap, temp_coef, temp_every, lam, out_scale, eps;
};

// Writes the step's keys [kv_heads][2 * head_dim] and values [kv_heads][value_dim] into their pages.
__global__ void diff_kv_write_kernel(const elem_t* __restrict__ k, long k_stride, const elem_t* __restrict__ v, long v_stride,
                                     elem_t* __restrict__ k_pages, elem_t* __restrict__ v_pages,
                                     const int32_t* __restrict__ block_table, int max_blocks,
                                     const int32_t* __restrict__ slots, const int32_t* __restrict__ positions, int kv_heads,
                                     int key_dim, int value_dim, int page_size) {
    const int m = blockIdx.x;
    const int pos = positions[m];
    const int block = pos / page_size, at = pos % page_size;
    const int page = block < max_blocks ? block_table[(size_t)slots[m] * max_blocks + block] : -1;
    if (page < 0) return;                      // (no page: nothing is written)
    for (int i = threadIdx.x; i < kv_heads * key_dim; i += blockDim.x) {
        const int g = i / key_dim, d = i % key_dim;
        k_pages[(((size_t)page * kv_heads + g) * page_size + at) * key_dim + d] = k[(size_t)m * k_stride + i];
    }
    for (int i = threadIdx.x; i < kv_heads * value_dim; i += blockDim.x) {
        const int g = i / value_dim, d = i % value_dim;
        v_pages[(((size_t)page * kv_heads + g) * page_size + at) * value_dim + d] = v[(size_t)m * v_stride + i];
    }
}

__device__ __forceinline__ float query_temperature(int pos, float coef, float every) {
    return coef != 0.f ? 1.0f + coef * logf(floorf((float)(pos + 1) / every) + 1.0f) : 1.0f;
}

__global__ __launch_bounds__(64) void diff_attention_partial_kernel(DiffArgs a) {
    __shared__ float q_lds[256];
    __shared__ float k_lds[TILE_KEYS * (DIM_CHUNK + 1)];
    __shared__ float p_lds[TILE_KEYS];
    __shared__ long long k_off[TILE_KEYS];
    __shared__ long long v_off[TILE_KEYS];
    const int m = blockIdx.x, hm = blockIdx.y, split = blockIdx.z;
    const int head = hm >> 1, map = hm & 1;
    const int lane = threadIdx.x;
    const int D = a.head_dim, V = a.value_dim;
    const int kvh = head / (a.q_heads / a.kv_heads);
    const int pos = a.positions[m], slot = a.slots[m];
    int kbegin = 0, kend = pos + 1;
    if (a.max_splits > 1) {
        kbegin = split * a.split_keys;
        kend = min(kend, (split + 1) * a.split_keys);
    }
    float* dst = a.partial + (((size_t)m * a.q_heads * 2 + hm) * a.max_splits + split) * (V + 2);
    if (kbegin >= kend) return;                // (a range beyond the token: the merge does not read it)
    for (int i = lane; i < D; i += 64) q_lds[i] = to_float(a.q[(size_t)m * a.q_stride + (size_t)hm * D + i]);
    const float factor = a.scale * query_temperature(pos, a.temp_coef, a.temp_every);
    float run_max = -INFINITY, run_sum = 0.f, acc[MAX_V_REGS];
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) acc[i] = 0.f;
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    for (int t0 = (kbegin / TILE_KEYS) * TILE_KEYS; t0 < kend; t0 += TILE_KEYS) {
        __syncthreads();
        {
            const int kp = t0 + lane;
            long long ko = -1, vo = -1;
            if (kp >= kbegin && kp < kend) {
                const int block = kp / a.page_size;
                const int page = block < a.max_blocks ? table[block] : -1;
                if (page >= 0) {
                    const long long row = ((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size;
                    ko = row * (2 * D) + (long long)map * D;
                    vo = row * V;
                }
            }
            k_off[lane] = ko;
            v_off[lane] = vo;
        }
        float s = 0.f;
        for (int dc = 0; dc < D; dc += DIM_CHUNK) {
            const int dw = min(DIM_CHUNK, D - dc);
            __syncthreads();
            for (int i = lane; i < TILE_KEYS * dw; i += 64) {
                const int key = i / dw, d = i % dw;
                const long long off = k_off[key];
                k_lds[key * (DIM_CHUNK + 1) + d] = off >= 0 ? to_float(a.k_pages[off + dc + d]) : 0.f;
            }
            __syncthreads();
            const float* kr = k_lds + lane * (DIM_CHUNK + 1);
            float part = 0.f;
            for (int d = 0; d < dw; ++d) part += q_lds[dc + d] * kr[d];
            s += part;
        }
        const bool valid = k_off[lane] >= 0;
        s *= factor;
        if (a.softcap > 0.f) s = a.softcap * tanhf(s / a.softcap);
        if (!valid) s = -INFINITY;
        const float new_max = fmaxf(run_max, wave_max(s));
        const float p = (valid && new_max > -INFINITY) ? expf(s - new_max) : 0.f;
        const float corr = new_max > -INFINITY ? expf(run_max - new_max) : 1.f;
        run_sum = run_sum * corr + wave_sum(p);
        run_max = new_max;
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) acc[i] *= corr;
        p_lds[lane] = p;
        __syncthreads();
        const int nkeys = min(TILE_KEYS, kend - t0);
        for (int key = 0; key < nkeys; ++key) {
            const long long off = v_off[key];
            if (off < 0) continue;
            const float pk = p_lds[key];
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) acc[i] += pk * to_float(a.v_pages[off + c]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c < V) dst[c] = acc[i];
    }
    if (lane == 0) {
        dst[V] = run_max;
        dst[V + 1] = run_sum;
    }
}

// One wavefront per (token, head): both maps merged over their key ranges, then the head's epilogue.
__global__ __launch_bounds__(64) void diff_attention_combine_kernel(DiffArgs a) {
    __shared__ float w_lds[COMBINE_MAX_SPLITS];
    __shared__ float l_lds[COMBINE_MAX_SPLITS];
    const int m = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int V = a.value_dim;
    const int pos = a.positions[m];
    const int n = a.max_splits > 1 ? min(a.max_splits - 1, pos / a.split_keys) + 1 : 1;
    float maps[2][MAX_V_REGS];
    for (int map = 0; map < 2; ++map) {
        const float* base = a.partial + ((size_t)m * a.q_heads * 2 + head * 2 + map) * a.max_splits * (V + 2);
        float gmax = -INFINITY;
        __syncthreads();
        for (int s = lane; s < n; s += 64) {
            const float smax = base[(size_t)s * (V + 2) + V];
            w_lds[s] = smax;
            l_lds[s] = base[(size_t)s * (V + 2) + V + 1];
            gmax = fmaxf(gmax, smax);
        }
        gmax = wave_max(gmax);
        __syncthreads();
        for (int s = lane; s < n; s += 64) {
            const float smax = w_lds[s];
            w_lds[s] = smax > -INFINITY ? expf(smax - gmax) : 0.f;
        }
        __syncthreads();
        float den = 0.f;
        for (int s = 0; s < n; ++s) den += w_lds[s] * l_lds[s];
        float num[MAX_V_REGS];
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) num[i] = 0.f;
        for (int s = 0; s < n; ++s) {
            const float w = w_lds[s];
            const float* p = base + (size_t)s * (V + 2);
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) num[i] += w * p[c];
            }
        }
#pragma unroll
        for (int i = 0; i < MAX_V_REGS; ++i) maps[map][i] = den != 0.f ? num[i] / den : 0.f;
    }
    float o[MAX_V_REGS], ss = 0.f;
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        o[i] = c < V ? maps[0][i] - a.lam * maps[1][i] : 0.f;
        ss += o[i] * o[i];
    }
    ss = wave_sum(ss);
    const float unit = a.out_scale / sqrtf(ss / (float)V + a.eps);
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c >= V) continue;
        float y = o[i] * unit;
        if (a.gate) y *= 1.0f / (1.0f + expf(-to_float(a.gate[(size_t)m * a.gate_stride + (size_t)head * V + c])));
        a.out[((size_t)m * a.q_heads + head) * V + c] = from_float<elem_t>(y);
    }
}

extern "C" {

int mlr_diff_kv_write(const void* k, long k_stride, const void* v, long v_stride, void* k_pages, void* v_pages,
                      const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions, int rows,
                      int kv_heads, int key_dim, int value_dim, int page_size, hipStream_t stream) {
    if (rows <= 0) return 0;
    diff_kv_write_kernel<<<rows, 256, 0, stream>>>((const elem_t*)k, k_stride, (const elem_t*)v, v_stride, (elem_t*)k_pages,
                                                   (elem_t*)v_pages, block_table, max_blocks, slots, positions, kv_heads,
                                                   key_dim, value_dim, page_size);
    return (int)hipGetLastError();
}

int mlr_diff_attention(const void* q, long q_stride, const void* k_pages, const void* v_pages, const int32_t* block_table,
                       int max_blocks, const int32_t* slots, const int32_t* positions, const void* gate, long gate_stride,
                       void* out, float* partial, int rows, int q_heads, int kv_heads, int head_dim, int value_dim,
                       int page_size, float scale, float softcap, float temp_coef, float temp_every, float lam,
                       float out_scale, float eps, int split_keys, int max_splits, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (head_dim > 256 || value_dim > 64 * MAX_V_REGS || q_heads % kv_heads != 0 || partial == nullptr) return -1;
    if (max_splits < 1) max_splits = 1;
    if (max_splits > 1 && (split_keys <= 0 || split_keys % TILE_KEYS != 0 || max_splits > COMBINE_MAX_SPLITS)) return -2;
    if (temp_coef != 0.f && !(temp_every > 0.f)) return -3;
    DiffArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, (const elem_t*)v_pages, block_table, slots, positions,
               (const elem_t*)gate, gate_stride, (elem_t*)out, partial, max_blocks, q_heads, kv_heads, head_dim, value_dim,
               page_size, split_keys, max_splits, scale, softcap, temp_coef, temp_every, lam, out_scale, eps};
    diff_attention_partial_kernel<<<dim3(rows, q_heads * 2, max_splits), 64, 0, stream>>>(a);
    int err = (int)hipGetLastError();
    if (err != 0) return err;
    diff_attention_combine_kernel<<<dim3(rows, q_heads), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
}

}  // extern "C"
