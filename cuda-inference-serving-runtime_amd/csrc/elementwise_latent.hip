// Row-wise kernels of layers with a centred norm, latent attention and an ungated feed-forward:
//
//   layer norm        (x - mean) / sqrt(var + eps) * w (+ b), var the mean of the squared deviations, float statistics,
//                     optional row gather
//   rms of a slice    columns [first, first + n) of float rows, RMS-normed with a weight, as a product's operand
//   latent keys       a row of the down-projection [c: rank | kr: rot_dim]: c RMS-normed with a weight, kr turned by the
//                     row's position, both written into the row's cache slot as ONE key head [c | kr | 0] of `pad`
//                     coordinates and one value head [c | 0] (transposed in its page); the rotated parts of the row's
//                     queries go to q_out[t, h, rank .. rank + rot_dim), the rest of a head's pad is zeroed
//   products a head   out[t, h, :] = a[t, h, :] . w[h]^T, optionally times sigmoid(gate[t, h]): the small matrices of a
//                     latent attention that differ from head to head
//   activation        gelu (erf or tanh form) of a row-major matrix
//
// Attention over such a cache is attention with one key/value head of `pad` coordinates: a query head is
// [Wuk_h^T q_h | rot(qr_h)], its score with [c | kr] is q_h . (Wuk_h c) + rot(qr_h) . kr, and the weighted sum of
// the value heads [c | 0] is the latent that Wuv_h turns into the head's result.
#include "common.h"

// ------------------------------------------------------------------------------------------------ layer norm
template <typename OUT>
__global__ void __launch_bounds__(256)
layernorm_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b,
                 OUT* __restrict__ out, const int* __restrict__ rows, int dim, float eps) {
    __shared__ float red[4];
    const int r = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[r] : r) * dim;
    float s = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) s += xr[i];
    const float mean = block_sum<256>(s, red) / dim;
    float q = 0.f;
    for (int i = threadIdx.x; i < dim; i += 256) {
        const float d = xr[i] - mean;
        q += d * d;
    }
    const float inv = rsqrtf(block_sum<256>(q, red) / dim + eps);
    OUT* o = out + (size_t)r * dim;
    for (int i = threadIdx.x; i < dim; i += 256) store_f32(o + i, (xr[i] - mean) * inv * w[i] + (b ? b[i] : 0.f));
}

// Rows of a multiple of four floats, at most 256 CH of them, 16-byte aligned: one wave a row, the row in registers (CH
// words of four floats a lane), no barrier; the statistics meet over the lanes.
template <typename OUT, int CH>
__global__ void __launch_bounds__(256)
layernorm_wave_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b,
                      OUT* __restrict__ out, const int* __restrict__ rows, int n_out, int dim, float eps) {
    typedef __attribute__((ext_vector_type(4))) float f32x4_t;
    const int r = blockIdx.x * 4 + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (r >= n_out) return;
    const f32x4_t* xr = (const f32x4_t*)(x + (size_t)(rows ? rows[r] : r) * dim);
    const int words = dim / 4;
    f32x4_t v[CH];
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int at = lane + WAVE * i;
        v[i] = at < words ? xr[at] : (f32x4_t){0.f, 0.f, 0.f, 0.f};
        s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    }
    const float mean = wave_sum(s) / dim;
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        if (lane + WAVE * i >= words) continue;
        v[i].x -= mean; v[i].y -= mean; v[i].z -= mean; v[i].w -= mean;
        q += (v[i].x * v[i].x + v[i].y * v[i].y) + (v[i].z * v[i].z + v[i].w * v[i].w);
    }
    const float inv = rsqrtf(wave_sum(q) / dim + eps);
#pragma unroll
    for (int i = 0; i < CH; ++i) {
        const int at = lane + WAVE * i;
        if (at >= words) continue;
        const f32x4_t ww = ((const f32x4_t*)w)[at];
        const f32x4_t bb = b ? ((const f32x4_t*)b)[at] : (f32x4_t){0.f, 0.f, 0.f, 0.f};
        const f32x4_t y = {v[i].x * inv * ww.x + bb.x, v[i].y * inv * ww.y + bb.y, v[i].z * inv * ww.z + bb.z, v[i].w * inv * ww.w + bb.w};
        if (sizeof(OUT) == 4) {
            ((f32x4_t*)((float*)out + (size_t)r * dim))[at] = y;
        } else {
            typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
            ((u32x2_t*)((bf16_t*)out + (size_t)r * dim))[at] = (u32x2_t){pack_bf16x2(y.x, y.y), pack_bf16x2(y.z, y.w)};
        }
    }
}

template <typename OUT>
static int launch_layernorm(const float* x, const float* w, const float* b, OUT* out, const int* rows, int n_out, int dim,
                            float eps, hipStream_t stream) {
    const bool aligned = dim % 4 == 0 && ((uintptr_t)x) % 16 == 0 && ((uintptr_t)w) % 16 == 0 && (!b || ((uintptr_t)b) % 16 == 0) &&
                         ((uintptr_t)out) % 16 == 0;
    const int per_lane = (dim / 4 + WAVE - 1) / WAVE;
    const unsigned blocks = (unsigned)((n_out + 3) / 4);
#define LN_WAVE(CH) layernorm_wave_kernel<OUT, CH><<<blocks, 256, 0, stream>>>(x, w, b, out, rows, n_out, dim, eps)
    if (aligned && per_lane <= 1) LN_WAVE(1);
    else if (aligned && per_lane <= 2) LN_WAVE(2);
    else if (aligned && per_lane <= 4) LN_WAVE(4);
    else if (aligned && per_lane <= 8) LN_WAVE(8);
    else if (aligned && per_lane <= 16) LN_WAVE(16);
    else layernorm_kernel<OUT><<<n_out, 256, 0, stream>>>(x, w, b, out, rows, dim, eps);
#undef LN_WAVE
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_layernorm(const float* x, const float* w, const float* b, void* out, const int* rows, int n_out,
                              int dim, float eps, int out_dtype, hipStream_t stream) {
    if (n_out <= 0) return 0;
    if (dim <= 0) return (int)hipErrorInvalidValue;
    if (out_dtype == DT_F32) return launch_layernorm<float>(x, w, b, (float*)out, rows, n_out, dim, eps, stream);
    return launch_layernorm<bf16_t>(x, w, b, (bf16_t*)out, rows, n_out, dim, eps, stream);
}

// ------------------------------------------------------------------------------------------------ rms of a slice
template <typename OUT>
__global__ void __launch_bounds__(256)
rms_slice_kernel(const float* __restrict__ x, int ld, int first, const float* __restrict__ w, OUT* __restrict__ out,
                 int n, float eps) {
    __shared__ float red[4];
    const float* xr = x + (size_t)blockIdx.x * ld + first;
    float q = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) q += xr[i] * xr[i];
    const float inv = rsqrtf(block_sum<256>(q, red) / n + eps);
    OUT* o = out + (size_t)blockIdx.x * n;
    for (int i = threadIdx.x; i < n; i += 256) store_f32(o + i, xr[i] * inv * w[i]);
}

extern "C" int cisr_rms_slice(const float* x, int ld, int first, const float* w, void* out, int rows, int n, float eps,
                              int out_dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (n <= 0 || first < 0 || first + n > ld) return (int)hipErrorInvalidValue;
    if (out_dtype == DT_F32) rms_slice_kernel<float><<<rows, 256, 0, stream>>>(x, ld, first, w, (float*)out, n, eps);
    else rms_slice_kernel<bf16_t><<<rows, 256, 0, stream>>>(x, ld, first, w, (bf16_t*)out, n, eps);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------------------ latent keys
struct LatentArgs {
    const float* down; int ld, first;        // down[t * ld + first + i]: i < rank the latent, then rot_dim coordinates
    const float* weight;                     // [rank]
    const void* q; int ldq;                  // q[t * ldq + h * (dim + rot_dim) + dim + i]: the part of a query that turns
    void* q_out;                             // [T, heads, pad]
    void* kcache; void* vcache;              // [pages, 1, page, pad], [pages, 1, pad, page]
    const int* positions; const int* slots;
    const float* cos; const float* sin;      // [max_pos, rot / 2]
    int heads, dim, rot_dim, rot, rank, pad, page, max_pos, interleaved;
    float eps;
};

// the two coordinates of pair j and their turned values; coordinates from `rot` on pass
__device__ __forceinline__ void pair_of(int j, int rot, int interleaved, int& a, int& b) {
    if (interleaved) { a = 2 * j; b = 2 * j + 1; }
    else { a = j; b = j + rot / 2; }
}

template <typename T>
__global__ void __launch_bounds__(256) latent_keys_kernel(LatentArgs p) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    const int pos = min(max(p.positions[t], 0), p.max_pos - 1), half = p.rot / 2;
    const float* cs = p.cos + (size_t)pos * half;
    const float* sn = p.sin + (size_t)pos * half;
    const float* row = p.down + (size_t)t * p.ld + p.first;
    const int slot = p.slots ? p.slots[t] : -1;
    float ss = 0.f;
    for (int i = tid; i < p.rank; i += 256) ss += row[i] * row[i];
    const float inv = rsqrtf(block_sum<256>(ss, red) / p.rank + p.eps);
    if (slot >= 0) {
        const size_t page = (size_t)(slot / p.page), in_page = (size_t)(slot % p.page);
        T* key = (T*)p.kcache + (page * p.page + in_page) * p.pad;
        T* val = (T*)p.vcache + page * p.pad * p.page + in_page;
        for (int i = tid; i < p.rank; i += 256) {
            const float c = row[i] * inv * p.weight[i];
            store_f32(key + i, c);
            store_f32(val + (size_t)i * p.page, c);
        }
        const float* kr = row + p.rank;
        for (int j = tid; j < half; j += 256) {
            int a, b;
            pair_of(j, p.rot, p.interleaved, a, b);
            const float u = kr[a], v = kr[b];
            store_f32(key + p.rank + a, u * cs[j] - v * sn[j]);
            store_f32(key + p.rank + b, v * cs[j] + u * sn[j]);
        }
        for (int i = p.rot + tid; i < p.rot_dim; i += 256) store_f32(key + p.rank + i, kr[i]);
        for (int i = p.rank + p.rot_dim + tid; i < p.pad; i += 256) store_f32(key + i, 0.f);
        for (int i = p.rank + tid; i < p.pad; i += 256) store_f32(val + (size_t)i * p.page, 0.f);
    }
    // the queries' turned parts and the zeros behind them
    const int tail = p.pad - p.rank;                // coordinates of a head of q_out that this kernel writes
    for (int idx = tid; idx < p.heads * tail; idx += 256) {
        const int h = idx / tail, i = idx % tail;
        const T* qr = (const T*)p.q + (size_t)t * p.ldq + (size_t)h * (p.dim + p.rot_dim) + p.dim;
        T* o = (T*)p.q_out + ((size_t)t * p.heads + h) * p.pad + p.rank;
        float y = 0.f;
        if (i < p.rot) {
            // coordinate i belongs to pair j as its first or its second member
            int j, first;
            if (p.interleaved) { j = i / 2; first = (i % 2 == 0); }
            else { j = i < half ? i : i - half; first = i < half; }
            int a, b;
            pair_of(j, p.rot, p.interleaved, a, b);
            const float u = load_f32(qr + a), v = load_f32(qr + b);
            y = first ? u * cs[j] - v * sn[j] : v * cs[j] + u * sn[j];
        } else if (i < p.rot_dim) {
            y = load_f32(qr + i);
        }
        store_f32(o + i, y);
    }
}

extern "C" int cisr_latent_keys(const float* down, int ld, int first, const float* weight, const void* q, int ldq,
                                void* q_out, void* kcache, void* vcache, const int* positions, const int* slots,
                                const float* cos, const float* sin, int rows, int heads, int dim, int rot_dim, int rot,
                                int rank, int pad, int page, int max_pos, int interleaved, float eps, int dtype,
                                hipStream_t stream) {
    if (rows <= 0) return 0;
    if (rot <= 0 || rot % 2 || rot > rot_dim || rank + rot_dim > pad || page <= 0 || max_pos <= 0 || first < 0 ||
        first + rank + rot_dim > ld || heads <= 0)
        return (int)hipErrorInvalidValue;
    LatentArgs p{down, ld, first, weight, q, ldq, q_out, kcache, vcache, positions, slots, cos, sin,
                 heads, dim, rot_dim, rot, rank, pad, page, max_pos, interleaved, eps};
    if (dtype == DT_F32) latent_keys_kernel<float><<<rows, 256, 0, stream>>>(p);
    else latent_keys_kernel<bf16_t><<<rows, 256, 0, stream>>>(p);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------------------ products a head
// out[t * ldo + h * out_head + n] = sigmoid?(gate[t * ldg + h]) * sum_k a[t * lda + h * a_head + k] * w[(h * N + n) * K + k]
// The plain form: a thread an output element, float sums in the order of k.
template <typename T>
__global__ void __launch_bounds__(256)
heads_product_kernel(const T* __restrict__ a, int lda, int a_head, const T* __restrict__ w, T* __restrict__ out, int ldo,
                     int out_head, const float* __restrict__ gate, int ldg, int heads, int N, int K) {
    const int n = blockIdx.x * 256 + threadIdx.x, h = blockIdx.y, t = blockIdx.z;
    if (n >= N) return;
    const T* ar = a + (size_t)t * lda + (size_t)h * a_head;
    const T* wr = w + ((size_t)h * N + n) * K;
    float acc = 0.f;
    for (int k = 0; k < K; ++k) acc += load_f32(ar + k) * load_f32(wr + k);
    if (gate) acc *= 1.0f / (1.0f + expf(-gate[(size_t)t * ldg + h]));
    store_f32(out + (size_t)t * ldo + (size_t)h * out_head + n, acc);
}

extern "C" int cisr_heads_product(const void* a, int lda, int a_head, const void* w, void* out, int ldo, int out_head,
                                  const float* gate, int ldg, int rows, int heads, int N, int K, int dtype,
                                  hipStream_t stream) {
    if (rows <= 0 || heads <= 0 || N <= 0) return 0;
    if (K <= 0 || heads > 65535) return (int)hipErrorInvalidValue;
    for (int r0 = 0; r0 < rows; r0 += 65535) {           // (the grid's third dimension holds at most 65,535 rows)
        const int n_rows = min(rows - r0, 65535);
        const dim3 grid((N + 255) / 256, heads, n_rows);
        if (dtype == DT_F32)
            heads_product_kernel<float><<<grid, 256, 0, stream>>>((const float*)a + (size_t)r0 * lda, lda, a_head, (const float*)w,
                                                                  (float*)out + (size_t)r0 * ldo, ldo, out_head,
                                                                  gate ? gate + (size_t)r0 * ldg : nullptr, ldg, heads, N, K);
        else
            heads_product_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a + (size_t)r0 * lda, lda, a_head, (const bf16_t*)w,
                                                                   (bf16_t*)out + (size_t)r0 * ldo, ldo, out_head,
                                                                   gate ? gate + (size_t)r0 * ldg : nullptr, ldg, heads, N, K);
        const int err = CISR_LAUNCH_CHECK();
        if (err) return err;
    }
    return 0;
}

// ------------------------------------------------------------------------------------------------ activation
// kind 0: the gelu with the error function; kind 1: its tanh form; kind 2: relu(z)^2 (unary_activation of common.h)
template <typename T>
__global__ void __launch_bounds__(256) gelu_kernel(const T* __restrict__ x, T* __restrict__ out, size_t n, int kind) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) store_f32(out + i, unary_activation(load_f32(x + i), kind + 1));
}

// out = act(x + bias[column]) for a product whose bias keeps the activation out of its epilogue; the sum is float
template <typename T>
__global__ void __launch_bounds__(256) bias_act_kernel(const T* __restrict__ x, const float* __restrict__ bias, T* __restrict__ out,
                                                       size_t n, int cols, int kind) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) store_f32(out + i, unary_activation(load_f32(x + i) + bias[i % cols], kind + 1));
}

extern "C" int cisr_bias_act(const void* x, const float* bias, void* out, long long n, int cols, int kind, int dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    if (kind < 0 || kind > 2 || cols <= 0 || !bias) return (int)hipErrorInvalidValue;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) bias_act_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, bias, (float*)out, (size_t)n, cols, kind);
    else bias_act_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, bias, (bf16_t*)out, (size_t)n, cols, kind);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_gelu(const void* x, void* out, long long n, int kind, int dtype, hipStream_t stream) {
    if (n <= 0) return 0;
    if (kind < 0 || kind > 2) return (int)hipErrorInvalidValue;
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) gelu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)x, (float*)out, (size_t)n, kind);
    else gelu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)x, (bf16_t*)out, (size_t)n, kind);
    return CISR_LAUNCH_CHECK();
}
