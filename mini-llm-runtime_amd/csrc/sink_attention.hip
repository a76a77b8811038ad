// Softmax attention with a sink and a mask rule over the paged cache, for mixers whose keys and values have
// sizes of their own, and the row kernels that prepare their queries, keys and values.
//
// A query at position p of a request sees the keys lo(p) .. p of the same request:
//   MASK_ALL     lo = 0
//   MASK_WINDOW  lo = max(0, p - size + 1)         (itself and the size - 1 tokens before it)
//   MASK_CHUNK   lo = floor(p / size) * size        (the keys of its own block of `size` positions)
// positions counted from the request's first token, never from where a step cut it.  The softmax's denominator
// holds one more summand, exp(sink[head]) (no key, no value, not scaled); sink == null: none.
// score = (q . k) * scale.  Scores, the softmax and its sums are 32-bit.
//
// Cache of one layer: key rows k_pages[page][kv_head][place in page][k_row] of which the first key_dim channels
// are the key, value rows v_pages[page][kv_head][place][v_row] of which the first value_dim channels are the
// value; both row-major.  The value rows may BE the key rows (v_pages == k_pages, v_row == k_row): a latent
// vector that serves as the first channels of the key and as the value.  Query head h reads kv head
// h / (q_heads / kv_heads).
//
// `sink_attention_kernel`: one wavefront per (token, head); tiles of 64 keys that start at multiples of 64 of the
// absolute position, so the order of a token's sums follows from its own position alone, never from the batch
// around it or from how its request was cut into steps.  The float engine's only attention, and the bfloat16
// engine's for sizes that the matrix-core kernel does not take.
// `sink_attention_tiles_kernel` (bfloat16): the same on the matrix cores, see there.
#include "common.h"

#define MASK_ALL 0
#define MASK_WINDOW 1
#define MASK_CHUNK 2

#define TILE_KEYS 64
#define DIM_CHUNK 64
#define MAX_KEY_DIM 2048
#define MAX_V_REGS 16           // value_dim <= 64 * MAX_V_REGS

struct SinkArgs {
    const elem_t* q; long q_stride;            // q[m * q_stride + head * key_dim + d]
    const elem_t* k_pages; long k_row;
    const elem_t* v_pages; long v_row;
    const int32_t* block_table; const int32_t* slots; const int32_t* positions;
    const float* sink;                         // [q_heads] or null
    elem_t* out; long out_stride;              // out[m * out_stride + head * value_dim + c]
    int max_blocks, q_heads, kv_heads, key_dim, value_dim, page_size, mask_kind, mask_size;
    float scale;
};

__device__ __forceinline__ int first_seen(int pos, int kind, int size) {
    if (kind == MASK_WINDOW) return max(0, pos - size + 1);
    if (kind == MASK_CHUNK) return (pos / size) * size;
    return 0;
}

__global__ __launch_bounds__(64) void sink_attention_kernel(SinkArgs a) {
    __shared__ float q_lds[MAX_KEY_DIM];
    __shared__ float k_lds[TILE_KEYS * (DIM_CHUNK + 1)];
    __shared__ float p_lds[TILE_KEYS];
    __shared__ long long row_of[TILE_KEYS];
    const int m = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int D = a.key_dim, V = a.value_dim;
    const int kvh = head / (a.q_heads / a.kv_heads);
    const int pos = a.positions[m], slot = a.slots[m];
    const int kbegin = first_seen(pos, a.mask_kind, a.mask_size), kend = pos + 1;
    for (int i = lane; i < D; i += 64) q_lds[i] = to_float(a.q[(size_t)m * a.q_stride + (size_t)head * D + i]);
    float run_max = -INFINITY, run_sum = 0.f, acc[MAX_V_REGS];
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) acc[i] = 0.f;
    const int32_t* table = a.block_table + (size_t)slot * a.max_blocks;
    for (int t0 = (kbegin / TILE_KEYS) * TILE_KEYS; t0 < kend; t0 += TILE_KEYS) {
        __syncthreads();
        {
            const int kp = t0 + lane;
            long long r = -1;
            if (kp >= kbegin && kp < kend) {
                const int block = kp / a.page_size;
                const int page = block < a.max_blocks ? table[block] : -1;
                if (page >= 0) r = ((long long)page * a.kv_heads + kvh) * a.page_size + kp % a.page_size;
            }
            row_of[lane] = r;
        }
        float s = 0.f;
        for (int dc = 0; dc < D; dc += DIM_CHUNK) {
            const int dw = min(DIM_CHUNK, D - dc);
            __syncthreads();
            for (int i = lane; i < TILE_KEYS * dw; i += 64) {
                const int key = i / dw, d = i % dw;
                const long long r = row_of[key];
                k_lds[key * (DIM_CHUNK + 1) + d] = r >= 0 ? to_float(a.k_pages[r * a.k_row + dc + d]) : 0.f;
            }
            __syncthreads();
            const float* kr = k_lds + lane * (DIM_CHUNK + 1);
            float part = 0.f;
            for (int d = 0; d < dw; ++d) part += q_lds[dc + d] * kr[d];
            s += part;
        }
        const bool valid = row_of[lane] >= 0;
        s = valid ? s * a.scale : -INFINITY;
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
            const long long r = row_of[key];
            if (r < 0) continue;
            const float pk = p_lds[key];
            const elem_t* vr = a.v_pages + r * a.v_row;
#pragma unroll
            for (int i = 0; i < MAX_V_REGS; ++i) {
                const int c = lane + 64 * i;
                if (c < V) acc[i] += pk * to_float(vr[c]);
            }
        }
    }
    // the sink: one more summand of the denominator
    float top = run_max, den = run_sum, scale_acc = 1.f;
    if (a.sink != nullptr) {
        const float sk = a.sink[head];
        top = fmaxf(run_max, sk);
        scale_acc = run_max > -INFINITY ? expf(run_max - top) : 0.f;
        den = run_sum * scale_acc + expf(sk - top);
    }
    const float inv = den > 0.f ? scale_acc / den : 0.f;
    elem_t* dst = a.out + (size_t)m * a.out_stride + (size_t)head * V;
#pragma unroll
    for (int i = 0; i < MAX_V_REGS; ++i) {
        const int c = lane + 64 * i;
        if (c < V) dst[c] = from_float<elem_t>(acc[i] * inv);
    }
}

// ---------------------------------------------------------------------------------------------------------
// Queries, keys and values of a grouped-query attention from the stacked projection's output
// proj[m] = [q_heads * key_dim | kv_heads * key_dim | kv_heads * value_dim]: the projection's bias added (null:
// none), q and k normed per head over key_dim (x / sqrt(mean(x^2) + eps) * weight, the weight shared by the
// heads; null: no norm), the first rot_dim channels of a head turned by the token's position in pairs
// (j, j + rot_dim / 2) with cos = table[p][j], sin = table[p][rot_dim / 2 + j] (table null: no rotation);
// q to q_out [m, q_heads * key_dim], k and v into their pages.  One wavefront a head; 32-bit throughout.
__global__ __launch_bounds__(64) void sink_qkv_prep_kernel(
    const elem_t* __restrict__ proj, long ld, const float* __restrict__ bias, elem_t* __restrict__ q_out,
    elem_t* __restrict__ k_pages, long k_row, elem_t* __restrict__ v_pages, long v_row,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ positions, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
    float eps, const float* __restrict__ rope, int rot_dim, int q_heads, int kv_heads, int key_dim, int value_dim,
    int page_size, int write_cache) {
    __shared__ float x_lds[MAX_KEY_DIM];
    const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[m], slot = slots[m];
    long long cache_row = -1;
    if (unit >= q_heads) {
        if (!write_cache) return;
        const int block = pos / page_size;
        const int page = block < max_blocks ? block_table[(size_t)slot * max_blocks + block] : -1;
        if (page < 0) return;                  // (no page: nothing is written)
        const int kvh = unit < q_heads + kv_heads ? unit - q_heads : unit - q_heads - kv_heads;
        cache_row = ((long long)page * kv_heads + kvh) * page_size + pos % page_size;
    }
    if (unit >= q_heads + kv_heads) {          // a value head: bias, into its page
        const long off = (long)(q_heads + kv_heads) * key_dim + (long)(unit - q_heads - kv_heads) * value_dim;
        for (int c = lane; c < value_dim; c += 64)
            v_pages[cache_row * v_row + c] =
                from_float<elem_t>(to_float(proj[(size_t)m * ld + off + c]) + (bias ? bias[off + c] : 0.f));
        return;
    }
    const long off = (long)unit * key_dim;
    const float* w = unit < q_heads ? q_norm_w : k_norm_w;
    float sum = 0.f;
    for (int d = lane; d < key_dim; d += 64) {
        const float x = to_float(proj[(size_t)m * ld + off + d]) + (bias ? bias[off + d] : 0.f);
        x_lds[d] = x;
        sum += x * x;
    }
    if (w != nullptr) {
        sum = wave_sum(sum);
        const float r = 1.0f / sqrtf(sum / (float)key_dim + eps);
        for (int d = lane; d < key_dim; d += 64) x_lds[d] = (x_lds[d] * r) * w[d];
    }
    __syncthreads();
    elem_t* dst = unit < q_heads ? q_out + ((size_t)m * q_heads + unit) * key_dim : k_pages + cache_row * k_row;
    const int half = rot_dim >> 1;
    const float* cs = rope ? rope + (size_t)pos * rot_dim : nullptr;
    for (int d = lane; d < key_dim; d += 64) {
        float y = x_lds[d];
        if (cs != nullptr && d < rot_dim) {
            const int j = d < half ? d : d - half;
            const float c = cs[j], s = cs[half + j];
            y = d < half ? turn_x(x_lds[d], x_lds[d + half], c, s) : turn_y(x_lds[d - half], x_lds[d], c, s);
        }
        dst[d] = from_float<elem_t>(y);
    }
}

// Latent attention's row work.  proj[m] = [heads * (dim + rot) | rank + rot]: per head `dim` plain and `rot`
// rotated query channels, then the latent part (`rank` channels) and the one rotated key part all heads share.
//   units 0 .. heads - 1: the head's rotated query channels, turned by the token's position (pairs
//     (j, j + rot / 2)), to q_out[m][head][rank .. rank + rot) -- the plain channels reach
//     q_out[m][head][0 .. rank) through the key up-projection, which is another kernel's work;
//   unit heads: the latent part normed over its `rank` channels (x / sqrt(mean(x^2) + eps) * weight) and the
//     rotated key part turned, into the token's cache row [rank + rot].
__global__ __launch_bounds__(64) void latent_prep_kernel(
    const elem_t* __restrict__ proj, long ld, elem_t* __restrict__ q_out, elem_t* __restrict__ pages, long row_width,
    const int32_t* __restrict__ block_table, int max_blocks, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ positions, const float* __restrict__ norm_w, float eps, const float* __restrict__ rope,
    int heads, int dim, int rot, int rank, int page_size, int write_cache) {
    const int m = blockIdx.x, unit = blockIdx.y, lane = threadIdx.x;
    const int pos = positions[m];
    const int half = rot >> 1;
    const float* cs = rope + (size_t)pos * rot;
    if (unit < heads) {
        const elem_t* src = proj + (size_t)m * ld + (size_t)unit * (dim + rot) + dim;
        elem_t* dst = q_out + ((size_t)m * heads + unit) * (rank + rot) + rank;
        for (int j = lane; j < half; j += 64) {
            const float u = to_float(src[j]), v = to_float(src[j + half]);
            dst[j] = from_float<elem_t>(turn_x(u, v, cs[j], cs[half + j]));
            dst[j + half] = from_float<elem_t>(turn_y(u, v, cs[j], cs[half + j]));
        }
        return;
    }
    if (!write_cache) return;
    const int block = pos / page_size;
    const int page = block < max_blocks ? block_table[(size_t)slots[m] * max_blocks + block] : -1;
    if (page < 0) return;
    elem_t* dst = pages + ((long long)page * page_size + pos % page_size) * row_width;
    const elem_t* src = proj + (size_t)m * ld + (size_t)heads * (dim + rot);
    float sum = 0.f;
    for (int d = lane; d < rank; d += 64) {
        const float x = to_float(src[d]);
        sum += x * x;
    }
    sum = wave_sum(sum);
    const float r = 1.0f / sqrtf(sum / (float)rank + eps);
    for (int d = lane; d < rank; d += 64) dst[d] = from_float<elem_t>((to_float(src[d]) * r) * norm_w[d]);
    for (int j = lane; j < half; j += 64) {
        const float u = to_float(src[rank + j]), v = to_float(src[rank + j + half]);
        dst[rank + j] = from_float<elem_t>(turn_x(u, v, cs[j], cs[half + j]));
        dst[rank + j + half] = from_float<elem_t>(turn_y(u, v, cs[j], cs[half + j]));
    }
}

extern "C" {

int mlr_sink_attention(const void* q, long q_stride, const void* k_pages, long k_row, const void* v_pages, long v_row,
                       const int32_t* block_table, int max_blocks, const int32_t* slots, const int32_t* positions,
                       const float* sink, void* out, long out_stride, int rows, int q_heads, int kv_heads, int key_dim,
                       int value_dim, int page_size, int mask_kind, int mask_size, float scale, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (key_dim > MAX_KEY_DIM || value_dim > 64 * MAX_V_REGS || q_heads > 65535 || kv_heads <= 0 ||
        q_heads % kv_heads != 0 || (mask_kind != MASK_ALL && mask_size <= 0))
        return -1;
    SinkArgs a{(const elem_t*)q, q_stride, (const elem_t*)k_pages, k_row, (const elem_t*)v_pages, v_row, block_table,
               slots, positions, sink, (elem_t*)out, out_stride, max_blocks, q_heads, kv_heads, key_dim, value_dim,
               page_size, mask_kind, mask_size, scale};
    sink_attention_kernel<<<dim3(rows, q_heads), 64, 0, stream>>>(a);
    return (int)hipGetLastError();
}

int mlr_sink_qkv_prep(const void* proj, long ld, const float* bias, void* q_out, void* k_pages, long k_row,
                      void* v_pages, long v_row, const int32_t* block_table, int max_blocks, const int32_t* slots,
                      const int32_t* positions, const float* q_norm_w, const float* k_norm_w, float eps,
                      const float* rope, int rot_dim, int rows, int q_heads, int kv_heads, int key_dim, int value_dim,
                      int page_size, int write_cache, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (key_dim > MAX_KEY_DIM || q_heads + 2 * kv_heads > 65535 || rot_dim > key_dim || (rot_dim & 1)) return -1;
    sink_qkv_prep_kernel<<<dim3(rows, q_heads + 2 * kv_heads), 64, 0, stream>>>(
        (const elem_t*)proj, ld, bias, (elem_t*)q_out, (elem_t*)k_pages, k_row, (elem_t*)v_pages, v_row, block_table,
        max_blocks, slots, positions, q_norm_w, k_norm_w, eps, rope, rot_dim, q_heads, kv_heads, key_dim, value_dim,
        page_size, write_cache);
    return (int)hipGetLastError();
}

int mlr_latent_prep(const void* proj, long ld, void* q_out, void* pages, long row_width, const int32_t* block_table,
                    int max_blocks, const int32_t* slots, const int32_t* positions, const float* norm_w, float eps,
                    const float* rope, int rows, int heads, int dim, int rot, int rank, int page_size, int write_cache,
                    hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads + 1 > 65535 || (rot & 1) || rot <= 0 || rope == nullptr) return -1;
    latent_prep_kernel<<<dim3(rows, heads + 1), 64, 0, stream>>>(
        (const elem_t*)proj, ld, (elem_t*)q_out, (elem_t*)pages, row_width, block_table, max_blocks, slots, positions,
        norm_w, eps, rope, heads, dim, rot, rank, page_size, write_cache);
    return (int)hipGetLastError();
}

}  // extern "C"
