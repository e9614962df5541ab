// Row-wise kernels of layers that norm after the sum, of an embedding with a hashed table of token pairs, and of
// attention that norms queries and keys over the whole projection:
//   x[r] = table[token_r] * scale + pairs[hash(previous token, token_r)]          (the last row of `pairs` at position 0)
//   x <- rmsnorm(alpha x + y * sigmoid(g + b)) * w     (y a row, or the weighted sum of `top` rows; the gate optional)
//   q, k normed over all heads at once, neighbouring coordinates turned by the position, q into a buffer of padded
//   heads, k and v into the pages of the cache
// Statistics and the residual stream are float; `T` is the storage type of activations (float or bf16).
#include "common.h"

// ------------------------------------------------------------------ embedding with a table of hashed token pairs
// One block a row.  The token before a segment's first row is the request's last token of the step before, kept in
// `last_token[state slot]`.  SINGLE: every segment has one row, and the thread that reads the kept token then stores
// the row's own; otherwise store_last_token_kernel runs afterwards.
template <typename TE, typename TH, bool SINGLE>
__global__ void __launch_bounds__(256)
embedding_pairs_kernel(const int* __restrict__ tokens, const int* __restrict__ positions, const int* __restrict__ seg_of_row,
                       const int* __restrict__ seg_start, const int* __restrict__ state_slots, int* last_token,
                       const TE* __restrict__ table, const TE* __restrict__ pairs, float* __restrict__ out, TH* __restrict__ cast,
                       int dim, int vocab, float scale, int buckets, unsigned long long mul_prev, unsigned long long mul_cur) {
    __shared__ int pair_row;
    const int row = blockIdx.x;
    int tok = tokens[row];
    tok = tok < 0 ? 0 : tok >= vocab ? vocab - 1 : tok;
    if (pairs != nullptr) {
        if (threadIdx.x == 0) {
            const int seg = seg_of_row[row];
            int at = buckets;                                   // a sequence's first token (and rows of no segment)
            if (seg >= 0) {
                const int slot = state_slots[seg];
                if (positions[row] > 0) {
                    const int prev = row > seg_start[seg] ? tokens[row - 1] : last_token[slot];
                    at = (int)(((unsigned long long)(prev < 0 ? 0 : prev) * mul_prev + (unsigned long long)tok * mul_cur) % (unsigned long long)buckets);
                }
                if (SINGLE) last_token[slot] = tok;
            }
            pair_row = at;
        }
        __syncthreads();
    }
    const TE* e = table + (size_t)tok * dim;
    const TE* p = pairs != nullptr ? pairs + (size_t)pair_row * dim : nullptr;
    for (int d = threadIdx.x; d < dim; d += 256) {
        float v = load_f32(e + d) * scale;
        if (p) v += load_f32(p + d);
        out[(size_t)row * dim + d] = v;
        if (cast) store_f32(cast + (size_t)row * dim + d, v);
    }
}

__global__ void store_last_token_kernel(const int* __restrict__ tokens, const int* __restrict__ seg_start,
                                        const int* __restrict__ state_slots, int* __restrict__ last_token, int segments, int vocab) {
    const int seg = blockIdx.x * blockDim.x + threadIdx.x;
    if (seg >= segments) return;
    const int first = seg_start[seg], end = seg_start[seg + 1];
    if (end <= first) return;                                  // (padding of a captured step)
    int tok = tokens[end - 1];
    last_token[state_slots[seg]] = tok < 0 ? 0 : tok >= vocab ? vocab - 1 : tok;
}

extern "C" int cisr_embedding_pairs(const int* tokens, const int* positions, const int* seg_of_row, const int* seg_start,
                                    const int* state_slots, int* last_token, const void* table, const void* pairs, float* out,
                                    void* cast, int rows, int segments, int dim, int vocab, float scale, int buckets,
                                    long long mul_prev, long long mul_cur, int single_rows, int table_dtype, int cast_dtype,
                                    hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || vocab <= 0 || (pairs && (buckets <= 0 || mul_prev < 0 || mul_cur < 0 || !last_token))) return (int)hipErrorInvalidValue;
#define EMB(TE, TH, S) embedding_pairs_kernel<TE, TH, S><<<rows, 256, 0, stream>>>(tokens, positions, seg_of_row, seg_start, state_slots, \
        last_token, (const TE*)table, (const TE*)pairs, out, (TH*)cast, dim, vocab, scale, buckets, (unsigned long long)mul_prev, (unsigned long long)mul_cur)
    if (table_dtype == DT_F32) { if (single_rows) EMB(float, float, true); else EMB(float, float, false); }
    else if (cast_dtype == DT_F32) { if (single_rows) EMB(bf16_t, float, true); else EMB(bf16_t, float, false); }
    else { if (single_rows) EMB(bf16_t, bf16_t, true); else EMB(bf16_t, bf16_t, false); }
#undef EMB
    int err = CISR_LAUNCH_CHECK();
    if (err || !pairs || single_rows || segments <= 0) return err;
    store_last_token_kernel<<<(segments + 63) / 64, 64, 0, stream>>>(tokens, seg_start, state_slots, last_token, segments, vocab);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ the norm after the sum, with a gated sublayer
// One block a row: x <- rmsnorm(alpha x + y' gate) w, y' = y[row] or sum_k yw[row, k] y[row * top + k], gate =
// sigmoid(g[row] + gb) or 1.  The sum waits in x between the two passes (a thread reads back what it wrote itself).
// `cast`: a copy of the new row in the activations' type, what the sublayers read next.
template <typename TH>
__global__ void __launch_bounds__(256)
gate_post_norm_kernel(float* __restrict__ x, const float* __restrict__ y, int top, const float* __restrict__ yw,
                      const float* __restrict__ g, int ldg, const float* __restrict__ gb, const float* __restrict__ w,
                      TH* __restrict__ cast, int dim, float eps, float alpha) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    float* xr = x + row * dim;
    float ss = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
        float v;
        if (yw) {
            v = 0.f;
            for (int k = 0; k < top; ++k) v += yw[row * top + k] * y[(row * top + k) * dim + d];
        } else {
            v = y[row * dim + d];
        }
        if (g) v *= 1.0f / (1.0f + expf(-(g[row * ldg + d] + (gb ? gb[d] : 0.f))));
        v += alpha * xr[d];
        xr[d] = v;
        ss += v * v;
    }
    const float rs = 1.0f / sqrtf(block_sum<256>(ss, red) / (float)dim + eps);
    for (int d = threadIdx.x; d < dim; d += 256) {
        const float v = xr[d] * rs * w[d];
        xr[d] = v;
        if (cast) store_f32(cast + row * dim + d, v);
    }
}

extern "C" int cisr_gate_post_norm(float* x, const float* y, int top, const float* yw, const float* g, int ldg, const float* gb,
                                   const float* w, void* cast, int rows, int dim, float eps, float alpha, int cast_dtype,
                                   hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || top < 1) return (int)hipErrorInvalidValue;
    if (cast_dtype == DT_F32) gate_post_norm_kernel<float><<<rows, 256, 0, stream>>>(x, y, top, yw, g, ldg, gb, w, (float*)cast, dim, eps, alpha);
    else gate_post_norm_kernel<bf16_t><<<rows, 256, 0, stream>>>(x, y, top, yw, g, ldg, gb, w, (bf16_t*)cast, dim, eps, alpha);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ queries and keys normed over the whole projection
// One block a row of a projection with float results [q: heads x dim | k: kv_heads x dim | v: kv_heads x vdim | ...]
// (`bias`: float over these columns, added first, or null): q and k are RMS-normed over all their heads at once (a
// weight an element), the first 2 `half` coordinates of every head turn by the position's angles (cos / sin float
// [max_pos, half]) in neighbouring pairs (2i, 2i + 1), or with `split_half` in pairs (i, i + half); q goes to q_out
// [T, heads * pad], k and v into the pages at `slots` as heads of `pad` coordinates, the rest zero (keys [pages,
// kv_heads, page_size, pad], values transposed in a page).  `value_norm`: each head's value is divided by its root mean
// square over vdim first (no weight).  has_kv 0: the row has queries only.
#define WN_MAX_KV_HEADS 256
template <typename T>
__global__ void __launch_bounds__(256)
whole_norm_rope_scatter_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bias, const float* __restrict__ qw,
                               const float* __restrict__ kw, const int* __restrict__ positions, const int* __restrict__ slots,
                               const float* __restrict__ cosines, const float* __restrict__ sines, int half, int max_pos,
                               T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache, int heads, int kv_heads, int dim,
                               int vdim, int pad, int page_size, float eps, int has_kv, int split_half, int value_norm) {
    __shared__ float red[4];
    __shared__ float rv[WN_MAX_KV_HEADS];
    const size_t row = blockIdx.x;
    const float* pr = proj + row * ld;
    const int nq = heads * dim, nk = kv_heads * dim;
    auto val = [&](int i) { return bias ? pr[i] + bias[i] : pr[i]; };
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) { const float v = val(i); sq += v * v; }
    const float rq = 1.0f / sqrtf(block_sum<256>(sq, red) / (float)nq + eps);
    float rk = 0.f;
    if (has_kv) {
        for (int i = threadIdx.x; i < nk; i += 256) { const float v = val(nq + i); sk += v * v; }
        rk = 1.0f / sqrtf(block_sum<256>(sk, red) / (float)nk + eps);
        if (value_norm) {
            const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
            for (int h = wave; h < kv_heads; h += 4) {
                float sv = 0.f;
                for (int c = lane; c < vdim; c += WAVE) { const float v = val(nq + nk + h * vdim + c); sv += v * v; }
                sv = wave_sum(sv);
                if (lane == 0) rv[h] = 1.0f / sqrtf(sv / (float)vdim + eps);
            }
            __syncthreads();
        }
    }
    int p = positions[row];
    p = p < 0 ? 0 : p >= max_pos ? max_pos - 1 : p;
    const float* cr = cosines + (size_t)p * half;
    const float* sr = sines + (size_t)p * half;
    // coordinate c of a head of the normed vector that starts at column `first` (weights wt), turned if it lies among
    // the turning ones
    auto turned = [&](int first, const float* wt, int base, int c, float r) {
        const float own = val(first + base + c) * r * wt[base + c];
        if (c >= 2 * half) return own;
        const int mate = split_half ? (c < half ? c + half : c - half) : c ^ 1;
        const bool second = split_half ? c >= half : (c & 1);
        const int pair = split_half ? (c < half ? c : c - half) : c >> 1;
        const float other = val(first + base + mate) * r * wt[base + mate];
        const float co = cr[pair], si = sr[pair];
        return second ? own * co + other * si : own * co - other * si;
    };
    // (blockIdx.y: with few rows several blocks share a row's outputs; each makes the row's statistics for itself)
    const int first = threadIdx.x + 256 * blockIdx.y, stride = 256 * gridDim.y;
    for (int i = first; i < heads * pad; i += stride) {
        const int h = i / pad, c = i % pad;
        store_f32(q_out + row * (size_t)(heads * pad) + i, c < dim ? turned(0, qw, h * dim, c, rq) : 0.f);
    }
    if (!has_kv) return;
    const int slot = slots[row];
    if (slot < 0) return;
    const size_t page = slot / page_size, off = slot % page_size;
    for (int i = first; i < kv_heads * pad; i += stride) {
        const int h = i / pad, c = i % pad;
        const float kv = c < dim ? turned(nq, kw, h * dim, c, rk) : 0.f;
        const float vv = c < vdim ? val(nq + nk + h * vdim + c) * (value_norm ? rv[h] : 1.0f) : 0.f;
        store_f32(kcache + ((page * kv_heads + h) * page_size + off) * pad + c, kv);
        store_f32(vcache + ((page * kv_heads + h) * pad + c) * page_size + off, vv);
    }
}

extern "C" int cisr_whole_norm_rope_scatter(const float* proj, int ld, const float* bias, const float* qw, const float* kw,
                                            const int* positions, const int* slots, const float* cosines, const float* sines, int half,
                                            int max_pos, void* q_out, void* kcache, void* vcache, int rows, int heads, int kv_heads,
                                            int dim, int vdim, int pad, int page_size, float eps, int has_kv, int split_half,
                                            int value_norm, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || dim > pad || vdim > pad || 2 * half > dim || half < 0 || heads <= 0 || (has_kv && (kv_heads <= 0 || page_size <= 0)) ||
        (value_norm && kv_heads > WN_MAX_KV_HEADS))
        return (int)hipErrorInvalidValue;
    const dim3 grid(rows, rows <= 128 ? 4 : 1);
    if (dtype == DT_F32)
        whole_norm_rope_scatter_kernel<float><<<grid, 256, 0, stream>>>(proj, ld, bias, qw, kw, positions, slots, cosines, sines, half, max_pos,
            (float*)q_out, (float*)kcache, (float*)vcache, heads, kv_heads, dim, vdim, pad, page_size, eps, has_kv, split_half, value_norm);
    else
        whole_norm_rope_scatter_kernel<bf16_t><<<grid, 256, 0, stream>>>(proj, ld, bias, qw, kw, positions, slots, cosines, sines, half, max_pos,
            (bf16_t*)q_out, (bf16_t*)kcache, (bf16_t*)vcache, heads, kv_heads, dim, vdim, pad, page_size, eps, has_kv, split_half, value_norm);
    return CISR_LAUNCH_CHECK();
}
