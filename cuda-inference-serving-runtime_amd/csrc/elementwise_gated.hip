// Row-wise kernels of layers that norm a sublayer's output before the residual sum, of feed-forwards with a
// clamped gate, and of attention that norms its queries and keys per head and gates its heads:
//   x += mult * rmsnorm(y) * w                      (also with y = (rmsnorm(a) wa + rmsnorm(b) wb) / 2 made on the way,
//                                                    and with the next norm of x made on the way)
//   act = g sigmoid(slope g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit)
//   q, k normed per head, q into a buffer of padded heads, k and v into the pages of the cache
//   out[t, h, :] = attn[t, h, :vdim] * sigmoid(gate[t, h])
// Statistics and the residual stream are float; `T` is the storage type of activations (float or bf16).
#include "common.h"

// ------------------------------------------------- norm of a sublayer's output, scaled, into the residual stream
// One block a row.  TWO: the row is half the sum of two rows, each normed over the width with a weight of its own; or,
// without those weights (wa null), the plain sum ca a + cb b of the two rows.
// With next_out the norm that reads the residual stream next is made on the way: next_out = rmsnorm(x) * next_w, or with
// next_w null the new row itself in the activations' type (for sublayers that read the stream as it is).
// KEEP: the row waits in LDS between the passes (rows of up to 16,384 floats); else it is read again.
template <bool TWO, bool KEEP, typename T>
__global__ void __launch_bounds__(256)
post_norm_add_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ wa,
                     const float* __restrict__ b, const float* __restrict__ wb, const float* __restrict__ w,
                     int dim, float eps, float mult, const float* __restrict__ next_w, float next_eps, T* __restrict__ next_out,
                     float ca, float cb, const float* __restrict__ bias_a) {
    __shared__ float red[4];
    extern __shared__ float kept[];
    const size_t row = blockIdx.x;
    const float* ar = a + row * dim;
    const float* br = TWO ? b + row * dim : nullptr;
    auto first = [&](int d) { return bias_a ? ar[d] + bias_a[d] : ar[d]; };     // (a bias a column that the product left out)
    float sa = 0.f, sb = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {
        const float u = first(d);
        sa += u * u;
        if (TWO) { const float v = br[d]; sb += v * v; }
        else if (KEEP) kept[d] = u;
    }
    float ra = 1.f, rb = 0.f;
    if (TWO) {
        ra = wa ? 0.5f / sqrtf(block_sum<256>(sa, red) / (float)dim + eps) : ca;
        rb = wa ? 0.5f / sqrtf(block_sum<256>(sb, red) / (float)dim + eps) : cb;
        sa = 0.f;
        for (int d = threadIdx.x; d < dim; d += 256) {
            const float y = first(d) * ra * (wa ? wa[d] : 1.0f) + br[d] * rb * (wa ? wb[d] : 1.0f);
            if (KEEP) kept[d] = y;
            sa += y * y;
        }
    }
    // (w null: the row is added as it is, times mult)
    const float scale = w ? mult / sqrtf(block_sum<256>(sa, red) / (float)dim + eps) : mult;
    float* xr = x + row * dim;
    float sn = 0.f;
    for (int d = threadIdx.x; d < dim; d += 256) {         // (a thread reads back only what it wrote itself)
        const float y = KEEP ? kept[d] : TWO ? first(d) * ra * (wa ? wa[d] : 1.0f) + br[d] * rb * (wa ? wb[d] : 1.0f) : first(d);
        const float xn = xr[d] + y * scale * (w ? w[d] : 1.0f);
        xr[d] = xn;
        if (KEEP) kept[d] = xn;
        sn += xn * xn;
    }
    if (next_out == nullptr) return;
    const float rs = next_w ? 1.0f / sqrtf(block_sum<256>(sn, red) / (float)dim + next_eps) : 1.0f;
    T* out = next_out + row * dim;
    for (int d = threadIdx.x; d < dim; d += 256) store_f32(out + d, (KEEP ? kept[d] : xr[d]) * rs * (next_w ? next_w[d] : 1.0f));
}

// The same for rows of up to 4,096 floats: a thread holds E elements of every operand in registers, so that all of a
// row's loads are on their way together (one trip to memory instead of one a pass).  slices_a / slices_b > 0: a (b) is
// a product that was cut along its inner size and left as partial sums [slices][rows][dim], added here in slice order.
template <bool TWO, int E, typename T>
__global__ void __launch_bounds__(256)
post_norm_add_short_kernel(float* __restrict__ x, const float* __restrict__ a, const float* __restrict__ wa,
                           const float* __restrict__ b, const float* __restrict__ wb, const float* __restrict__ w,
                           int dim, float eps, float mult, const float* __restrict__ next_w, float next_eps, T* __restrict__ next_out,
                           int slices_a, int slices_b, float ca, float cb, const float* __restrict__ bias_a) {
    __shared__ float red[4];
    const size_t row = blockIdx.x;
    float va[E], vb[E], vx[E], vw[E], vwa[E], vwb[E], vn[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int d = threadIdx.x + 256 * e;
        const bool in = d < dim;
        const int dd = in ? d : 0;
        va[e] = in ? a[row * dim + dd] : 0.f;
        vx[e] = in ? x[row * dim + dd] : 0.f;
        vw[e] = w ? w[dd] : 1.f;
        vn[e] = next_w ? next_w[dd] : 1.f;
        if (TWO) { vb[e] = in ? b[row * dim + dd] : 0.f; vwa[e] = wa ? wa[dd] : 1.f; vwb[e] = wa ? wb[dd] : 1.f; }
    }
    // the further slices of a cut product, four slices' loads on their way at a time, added in slice order
    auto add_slices = [&](float (&v)[E], const float* parts, int slices) {
        for (int s0 = 1; s0 < slices; s0 += 4) {
            float more[4][E];
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const int d = threadIdx.x + 256 * e;
                    more[j][e] = (s0 + j < slices && d < dim) ? parts[((size_t)(s0 + j) * gridDim.x + row) * dim + d] : 0.f;
                }
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int e = 0; e < E; ++e) v[e] += more[j][e];
        }
    };
    if (slices_a > 1) add_slices(va, a, slices_a);
    if (TWO && slices_b > 1) add_slices(vb, b, slices_b);
    if (bias_a) {                                             // (a bias a column that the product left out)
#pragma unroll
        for (int e = 0; e < E; ++e) { const int d = threadIdx.x + 256 * e; if (d < dim) va[e] += bias_a[d]; }
    }
    float sa = 0.f, sb = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) { sa += va[e] * va[e]; if (TWO) sb += vb[e] * vb[e]; }
    if (TWO) {
        const float ra = wa ? 0.5f / sqrtf(block_sum<256>(sa, red) / (float)dim + eps) : ca;
        const float rb = wa ? 0.5f / sqrtf(block_sum<256>(sb, red) / (float)dim + eps) : cb;
        sa = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) { va[e] = va[e] * ra * vwa[e] + vb[e] * rb * vwb[e]; sa += va[e] * va[e]; }
    }
    const float scale = w ? mult / sqrtf(block_sum<256>(sa, red) / (float)dim + eps) : mult;
    float sn = 0.f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int d = threadIdx.x + 256 * e;
        vx[e] += va[e] * scale * vw[e];
        if (d < dim) { x[row * dim + d] = vx[e]; sn += vx[e] * vx[e]; }
    }
    if (next_out == nullptr) return;
    const float rs = next_w ? 1.0f / sqrtf(block_sum<256>(sn, red) / (float)dim + next_eps) : 1.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int d = threadIdx.x + 256 * e;
        if (d < dim) store_f32(next_out + row * dim + d, vx[e] * rs * vn[e]);
    }
}

template <bool TWO, typename T>
static void launch_post_norm_add(float* x, const float* a, const float* wa, const float* b, const float* wb, const float* w,
                                 int rows, int dim, float eps, float mult, const float* next_w, float next_eps, T* next_out,
                                 int slices_a, int slices_b, float ca, float cb, const float* bias_a, hipStream_t stream) {
#define SHORT(E) post_norm_add_short_kernel<TWO, E, T><<<rows, 256, 0, stream>>>(x, a, wa, b, wb, w, dim, eps, mult, next_w, next_eps, next_out, slices_a, slices_b, ca, cb, bias_a)
    if (dim <= 1024) SHORT(4);
    else if (dim <= 2048) SHORT(8);
    else if (dim <= 4096) SHORT(16);
#undef SHORT
    else if (dim <= 16384) post_norm_add_kernel<TWO, true, T><<<rows, 256, (size_t)dim * sizeof(float), stream>>>(x, a, wa, b, wb, w, dim, eps, mult, next_w, next_eps, next_out, ca, cb, bias_a);
    else post_norm_add_kernel<TWO, false, T><<<rows, 256, 0, stream>>>(x, a, wa, b, wb, w, dim, eps, mult, next_w, next_eps, next_out, ca, cb, bias_a);
}

extern "C" int cisr_post_norm_add(float* x, const float* a, const float* wa, const float* b, const float* wb,
                                  const float* w, int rows, int dim, float eps, float mult, const float* next_w, float next_eps,
                                  void* next_out, int next_dtype, int slices_a, int slices_b, float ca, float cb, const float* bias_a,
                                  hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || (b != nullptr && ((wa == nullptr) != (wb == nullptr))) || (next_w != nullptr && next_out == nullptr) ||
        slices_a < 0 || slices_b < 0 || ((slices_a > 0 || slices_b > 0) && dim > 4096))    // (partial sums: the kernel of short rows)
        return (int)hipErrorInvalidValue;
    if (next_dtype == DT_F32) {
        if (b) launch_post_norm_add<true, float>(x, a, wa, b, wb, w, rows, dim, eps, mult, next_w, next_eps, (float*)next_out, slices_a, slices_b, ca, cb, bias_a, stream);
        else launch_post_norm_add<false, float>(x, a, nullptr, nullptr, nullptr, w, rows, dim, eps, mult, next_w, next_eps, (float*)next_out, slices_a, slices_b, ca, cb, bias_a, stream);
    } else {
        if (b) launch_post_norm_add<true, bf16_t>(x, a, wa, b, wb, w, rows, dim, eps, mult, next_w, next_eps, (bf16_t*)next_out, slices_a, slices_b, ca, cb, bias_a, stream);
        else launch_post_norm_add<false, bf16_t>(x, a, nullptr, nullptr, nullptr, w, rows, dim, eps, mult, next_w, next_eps, (bf16_t*)next_out, slices_a, slices_b, ca, cb, bias_a, stream);
    }
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ clamped gated activation
// gu[r] = [gate (inter) | up (inter)]; arithmetic in float.
template <typename T>
__global__ void glu_clamped_kernel(const T* __restrict__ gu, T* __restrict__ act, int inter, size_t n,
                                   float limit, float slope, float shift) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const size_t row = i / inter;
    const int col = (int)(i % inter);
    const T* base = gu + row * (size_t)(2 * inter);
    const float g = fminf(load_f32(base + col), limit);
    const float u = fminf(fmaxf(load_f32(base + inter + col), -limit), limit);
    store_f32(act + i, g / (1.0f + expf(-slope * g)) * (u + shift));
}

// the same for bf16, eight elements a thread with 16-byte accesses (inter % 8 == 0, aligned pointers)
__global__ void __launch_bounds__(256)
glu_clamped_bf16x8_kernel(const bf16_t* __restrict__ gu, bf16_t* __restrict__ act, int inter8, size_t n8, GateLaw law) {
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const size_t row = i / inter8;
    const int col = (int)(i % inter8) * 8;
    const bf16_t* base = gu + row * (size_t)(16 * inter8);
    const u32x4_t g = *(const u32x4_t*)(base + col), u = *(const u32x4_t*)(base + 8 * inter8 + col);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t out[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
        out[k] = pack_bf16x2(gated_activation(__uint_as_float(gw[k] << 16), __uint_as_float(uw[k] << 16), law),
                             gated_activation(__uint_as_float(gw[k] & 0xffff0000u), __uint_as_float(uw[k] & 0xffff0000u), law));
    *(u32x4_t*)(act + i * 8) = (u32x4_t){out[0], out[1], out[2], out[3]};
}

extern "C" int cisr_glu_clamped(const void* gu, void* act, int rows, int inter, float limit, float slope, float shift,
                                int dtype, hipStream_t stream) {
    const size_t n = (size_t)rows * inter;
    if (n == 0) return 0;
    if (dtype == DT_BF16 && limit > 0.f && inter % 8 == 0 && ((uintptr_t)gu) % 16 == 0 && ((uintptr_t)act) % 16 == 0) {
        const size_t n8 = n / 8;
        glu_clamped_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)act, inter / 8, n8,
                                                                                  GateLaw{limit, slope, shift});
        return CISR_LAUNCH_CHECK();
    }
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) glu_clamped_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, (float*)act, inter, n, limit, slope, shift);
    else glu_clamped_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)act, inter, n, limit, slope, shift);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------- per-head norm of queries and keys + scatter into the pages
// A wave a (token row, head); a block holds four heads of a row.  The row of the fused projection is [q: heads x dim |
// k: kv_heads x dim | v: kv_heads x vdim | ...].  Queries go to q_out [T, heads, pad] (coordinates dim..pad-1 zero),
// keys to kcache [pages, kv_heads, page_size, pad] (likewise), values transposed to vcache [pages, kv_heads, pad,
// page_size] (coordinates vdim..pad-1 zero): heads of `pad` coordinates are what the attention kernels read.
// wq / wk null: that side is not normed.
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_scatter_kernel(const T* __restrict__ qkv, int ld, const float* __restrict__ wq, const float* __restrict__ wk,
                       T* __restrict__ q_out, T* __restrict__ kcache, T* __restrict__ vcache,
                       const int* __restrict__ slots, int heads, int kv_heads, int dim, int vdim, int pad,
                       int page_size, float eps) {
    const int row = blockIdx.x, wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const T* src = qkv + (size_t)row * ld;
    const int slot = slots ? slots[row] : -1;
    const int items = heads + 2 * kv_heads;
    for (int item = blockIdx.y * 4 + wave; item < items; item += 4 * gridDim.y) {
        if (item < heads + kv_heads) {
            const bool is_q = item < heads;
            const int head = is_q ? item : item - heads;
            if (!is_q && slot < 0) continue;
            const T* v = src + (size_t)item * dim;         // (queries and keys have the same size: one run of heads)
            const float* w = is_q ? wq : wk;
            float vals[4], ss = 0.f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = lane + WAVE * i;
                vals[i] = d < dim ? load_f32(v + d) : 0.f;
                ss += vals[i] * vals[i];
            }
            const float scale = w ? 1.0f / sqrtf(wave_sum(ss) / (float)dim + eps) : 1.0f;
            T* dst = is_q ? q_out + ((size_t)row * heads + head) * pad
                          : kcache + (((size_t)(slot / page_size) * kv_heads + head) * page_size + slot % page_size) * pad;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = lane + WAVE * i;
                if (d < pad) store_f32(dst + d, d < dim ? vals[i] * scale * (w ? w[d] : 1.0f) : 0.f);
            }
        } else {
            if (slot < 0) continue;
            const int head = item - heads - kv_heads;
            const T* v = src + (size_t)(heads + kv_heads) * dim + (size_t)head * vdim;
            T* dst = vcache + ((size_t)(slot / page_size) * kv_heads + head) * pad * page_size + slot % page_size;
            for (int d = lane; d < pad; d += WAVE) store_f32(dst + (size_t)d * page_size, d < vdim ? load_f32(v + d) : 0.f);
        }
    }
}

extern "C" int cisr_qk_norm_scatter(const void* qkv, int ld, const float* wq, const float* wk, void* q_out, void* kcache,
                                    void* vcache, const int* slots, int rows, int heads, int kv_heads, int dim, int vdim,
                                    int pad, int page_size, float eps, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || vdim <= 0 || dim > pad || vdim > pad || pad > 256 || page_size <= 0 ||
        ld < (heads + kv_heads) * dim + kv_heads * vdim)
        return (int)hipErrorInvalidValue;
    const dim3 grid(rows, min((heads + 2 * kv_heads + 3) / 4, 65535));
    if (dtype == DT_F32)
        qk_norm_scatter_kernel<float><<<grid, 256, 0, stream>>>((const float*)qkv, ld, wq, wk, (float*)q_out, (float*)kcache,
            (float*)vcache, slots, heads, kv_heads, dim, vdim, pad, page_size, eps);
    else
        qk_norm_scatter_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)qkv, ld, wq, wk, (bf16_t*)q_out, (bf16_t*)kcache,
            (bf16_t*)vcache, slots, heads, kv_heads, dim, vdim, pad, page_size, eps);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ one gate a head
// out[t, h, d] = attn[t, h, d] * sigmoid(gate[t * ld_gate + h]) for d < vdim; attn has heads of `pad` coordinates.
template <typename T>
__global__ void head_gate_kernel(const T* __restrict__ attn, const T* __restrict__ gate, int ld_gate,
                                 T* __restrict__ out, int heads, int vdim, int pad, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const int d = (int)(i % vdim);
    const size_t th = i / vdim;
    const int h = (int)(th % heads);
    const size_t t = th / heads;
    const float g = gate ? 1.0f / (1.0f + expf(-load_f32(gate + t * ld_gate + h))) : 1.0f;
    store_f32(out + i, load_f32(attn + th * pad + d) * g);
}

// the same for bf16 with vdim and pad multiples of eight: eight elements a thread, 16-byte accesses
__global__ void __launch_bounds__(256)
head_gate_bf16x8_kernel(const bf16_t* __restrict__ attn, const bf16_t* __restrict__ gate, int ld_gate, bf16_t* __restrict__ out,
                        int heads, int vdim8, int pad, size_t n8) {
    typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n8) return;
    const int d8 = (int)(i % vdim8);
    const size_t th = i / vdim8;
    const int h = (int)(th % heads);
    const size_t t = th / heads;
    const float g = gate ? 1.0f / (1.0f + expf(-bf16_to_f32(gate[t * ld_gate + h]))) : 1.0f;
    const u32x4_t a = *(const u32x4_t*)(attn + th * pad + d8 * 8);
    const uint32_t aw[4] = {a.x, a.y, a.z, a.w};
    uint32_t o[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) o[k] = pack_bf16x2(__uint_as_float(aw[k] << 16) * g, __uint_as_float(aw[k] & 0xffff0000u) * g);
    *(u32x4_t*)(out + i * 8) = (u32x4_t){o[0], o[1], o[2], o[3]};
}

extern "C" int cisr_head_gate(const void* attn, const void* gate, int ld_gate, void* out, int rows, int heads, int vdim,
                              int pad, int dtype, hipStream_t stream) {
    const size_t n = (size_t)rows * heads * vdim;
    if (n == 0) return 0;
    if (vdim > pad) return (int)hipErrorInvalidValue;
    if (dtype == DT_BF16 && vdim % 8 == 0 && pad % 8 == 0 && ((uintptr_t)attn) % 16 == 0 && ((uintptr_t)out) % 16 == 0) {
        const size_t n8 = n / 8;
        head_gate_bf16x8_kernel<<<(unsigned)((n8 + 255) / 256), 256, 0, stream>>>((const bf16_t*)attn, (const bf16_t*)gate, ld_gate,
                                                                                (bf16_t*)out, heads, vdim / 8, pad, n8);
        return CISR_LAUNCH_CHECK();
    }
    const unsigned blocks = (unsigned)((n + 255) / 256);
    if (dtype == DT_F32) head_gate_kernel<float><<<blocks, 256, 0, stream>>>((const float*)attn, (const float*)gate, ld_gate, (float*)out, heads, vdim, pad, n);
    else head_gate_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)attn, (const bf16_t*)gate, ld_gate, (bf16_t*)out, heads, vdim, pad, n);
    return CISR_LAUNCH_CHECK();
}
