// Attention whose scores are mixed over the heads before the softmax, over the paged cache: one block a token row,
// all query heads of the row together.
//
//   raw_g(j)  = q_g . k_kv(g)(j)                                   for every query head g and visible key j
//   s_h(j)    = sum_g mix[h, g] temp[g] scale raw_g(j)             (the heads' scores talk to each other)
//   w_h(j)    = exp(s_h(j)) / (exp(sink_h) + sum_j' exp(s_h(j')))  (a sink: a term of the denominator without a key)
//   out_h     = sum_j w_h(j) v_kv(h)(j)    [times sigmoid(gate) element by element]
//
// A row at position p sees the keys lo..p of its request: lo = (p / chunk) chunk with `chunk` > 0 (blocks of positions
// counted from 0 that see only themselves), p - window + 1 with `window` > 0, else 0.  Its own key is in the cache before
// this kernel runs.  Exact float arithmetic on float or bf16 storage (scores, the mix, the softmax and the sums are
// float); the pages hold heads of `pad` coordinates whose rest is zero (keys [pages, kv_heads, page_size, pad], values
// transposed in a page), queries come as [rows, heads * pad].
//
// Keys are walked 64 at a time, tiles at absolute multiples of 64: (1) a thread a (key head, key) makes the raw scores
// of the head's group, 16 bytes of the key row a load; (2) a thread a (head, key) mixes; (3) a wave a head moves the
// running maximum and denominator; (4) a thread an output coordinate (E of them in registers) adds the tile's values,
// eight keys of a transposed value page a load where pages hold a multiple of eight keys.  With `splits` > 1 that
// many blocks share a row's tiles (steps of few rows: one block a row leaves the GPU empty) and a small kernel merges.
#include "common.h"

#define TK_KEYS 64

struct TalkArgs {
    const void* q; int q_row_stride;
    const void* kcache; const void* vcache;
    const int* tables; const int* seg_of_row; const int* positions;
    const float* mix; const float* temp; const float* sink;
    const float* gate; int ldg;
    void* out;
    int heads, kv_heads, vdim, pad, page_size, width, window, chunk;
    float scale;
    int splits; float* part_o; float* part_ml;      // splits > 1: block (row, s) walks the tiles s, s + splits, ... and leaves sums
};

__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16_t* p, float (&v)[8]) {
    const uint4 a = *(const uint4*)p;
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { v[2 * i] = __uint_as_float(w[i] << 16); v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
}

template <typename T, int E>
__global__ void __launch_bounds__(256)
attn_talking_kernel(TalkArgs p) {
    extern __shared__ float lds[];
    const int H = p.heads, G = p.kv_heads, pad = p.pad, P = p.page_size, group = H / G;
    float* qs = lds;                          // [H, pad]
    float* mixw = qs + H * pad;               // [H, H]: mix[h, g] temp[g] scale
    float* raw = mixw + H * H;                // [H, 64]
    float* pw = raw + H * TK_KEYS;            // [H, 64]
    float* run_m = pw + H * TK_KEYS;          // [H]
    float* run_l = run_m + H;                 // [H]
    float* alpha = run_l + H;                 // [H]
    int* pg = (int*)(alpha + H);              // [64]: the page of a key of the tile (-1: not visible)
    int* po = pg + TK_KEYS;                   // [64]: its place in the page

    const int row = blockIdx.x, tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int seg = p.seg_of_row[row];
    const int n_out = H * p.vdim;
    T* out = (T*)p.out + (size_t)row * n_out;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.f;
    // Which output a thread's e-th accumulator is: coordinate (tid + 256 e) of the row as it lies in memory; or, where
    // the sizes allow (value heads that divide 256 and head counts that divide by 256 / vdim), one coordinate d of
    // consecutive heads, so that heads of one group follow each other and share the loads of their values.
    const int lanes_of_d = 256 / p.vdim;
    const bool packed = 256 % p.vdim == 0 && H % lanes_of_d == 0 && H / lanes_of_d <= E;
    const int heads_here = packed ? H / lanes_of_d : 0;
    auto owned = [&](int e) { return packed ? (e < heads_here ? ((tid / p.vdim) * heads_here + e) * p.vdim + tid % p.vdim : n_out) : tid + 256 * e; };
    int begin = 0, end = 0;
    if (seg >= 0) {
        const int pos = p.positions[row];
        end = pos + 1;
        begin = p.chunk > 0 ? (pos / p.chunk) * p.chunk : (p.window > 0 && end > p.window) ? end - p.window : 0;
    }
    const int split = blockIdx.y, S = p.splits;
    if (begin >= end) {
        if (S > 1) {                                  // (nothing to merge: every block along the keys says so)
            for (int h = tid; h < H; h += 256) {
                const size_t part = ((size_t)row * H + h) * S + split;
                p.part_ml[part * 2] = -INFINITY; p.part_ml[part * 2 + 1] = 0.f;
            }
            return;
        }
#pragma unroll
        for (int e = 0; e < E; ++e) { const int i = owned(e); if (i < n_out) store_f32(out + i, 0.f); }
        return;
    }
    const T* qr = (const T*)p.q + (size_t)row * p.q_row_stride;
    for (int i = tid; i < H * pad; i += 256) qs[i] = load_f32(qr + i);
    for (int i = tid; i < H * H; i += 256) mixw[i] = p.mix[i] * (p.temp ? p.temp[i % H] : 1.0f) * p.scale;
    for (int h = tid; h < H; h += 256) {
        const bool sunk = p.sink && split == 0;           // the sink: a key of score sink_h and no value; it counts once
        run_m[h] = sunk ? p.sink[h] : -INFINITY;
        run_l[h] = sunk ? 1.0f : 0.f;
    }
    const int* table = p.tables + (size_t)seg * p.width;
    const T* kc = (const T*)p.kcache;
    const T* vc = (const T*)p.vcache;
    const bool by8 = P % 8 == 0;
    for (int base = begin / TK_KEYS * TK_KEYS + split * TK_KEYS; base < end; base += S * TK_KEYS) {
        __syncthreads();                      // (the tile before is done with pg, po, pw, alpha; the first: qs, mixw are there)
        if (tid < TK_KEYS) {
            const int t = base + tid;
            const bool seen = t >= begin && t < end;
            pg[tid] = seen ? table[t / P] : -1;
            po[tid] = t % P;
        }
        __syncthreads();
        // (1) raw scores of a key head's group of query heads, four heads at a time
        for (int item = tid; item < G * TK_KEYS; item += 256) {
            const int c = item / TK_KEYS, j = item % TK_KEYS;
            if (pg[j] < 0) continue;
            const T* kr = kc + (((size_t)pg[j] * G + c) * P + po[j]) * pad;
            for (int g0 = 0; g0 < group; g0 += 4) {
                float dot[4] = {0.f, 0.f, 0.f, 0.f};
                const float* q0 = qs + (size_t)(c * group + g0) * pad;
                for (int d0 = 0; d0 < pad; d0 += 64) {             // 64 coordinates a trip: eight loads on their way together
                    float kv[8][8];
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        if (d0 + 8 * w < pad) load8(kr + d0 + 8 * w, kv[w]);
                    }
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        const int d = d0 + 8 * w;
                        if (d >= pad) continue;
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            if (g0 + u < group) {
                                const float* qh = q0 + u * pad + d;
#pragma unroll
                                for (int i = 0; i < 8; ++i) dot[u] += qh[i] * kv[w][i];
                            }
                        }
                    }
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) if (g0 + u < group) raw[(c * group + g0 + u) * TK_KEYS + j] = dot[u];
            }
        }
        __syncthreads();
        // (2) the mix over the heads
        for (int item = tid; item < H * TK_KEYS; item += 256) {
            const int h = item / TK_KEYS, j = item % TK_KEYS;
            float s = -INFINITY;
            if (pg[j] >= 0) {
                s = 0.f;
                for (int g = 0; g < H; ++g) s += mixw[h * H + g] * raw[g * TK_KEYS + j];
            }
            pw[item] = s;
        }
        __syncthreads();
        // (3) running maximum and denominator, a wave a head
        for (int h = wave; h < H; h += 4) {
            const float s = pw[h * TK_KEYS + lane];
            const float m_old = run_m[h];
            const float m_new = fmaxf(m_old, wave_max(s));          // finite: the tile has a visible key
            const float w = expf(s - m_new);                        // exp(-inf) = 0
            const float a = expf(m_old - m_new);
            const float l = run_l[h] * a + wave_sum(w);
            pw[h * TK_KEYS + lane] = w;
            if (lane == 0) { run_m[h] = m_new; run_l[h] = l; alpha[h] = a; }
        }
        __syncthreads();
        // (4) the values
        float vv[8][8];
        bool there[8];
        int c_held = -1, d_held = -1;                            // the key head and coordinate whose values vv holds
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int i = owned(e);
            if (i >= n_out) continue;
            const int h = i / p.vdim, d = i % p.vdim, c = h / group;
            float a = acc[e] * alpha[h];
            const float* wr = pw + h * TK_KEYS;
            if (by8) {
                // the tile's eight groups of eight keys: all loads on their way before the first is used; the values
                // stay for the next accumulator if that is a head of the same group
                if (c != c_held || d != d_held) {
                    c_held = c; d_held = d;
#pragma unroll
                    for (int w = 0; w < 8; ++w) {
                        const int j = 8 * w;
                        int page = -1;
#pragma unroll
                        for (int u = 0; u < 8; ++u) page = max(page, pg[j + u]);      // (eight keys from a multiple of eight: one page)
                        there[w] = page >= 0;
                        if (there[w]) load8(vc + (((size_t)page * G + c) * pad + d) * P + po[j], vv[w]);
                    }
                }
#pragma unroll
                for (int w = 0; w < 8; ++w) {
                    if (!there[w]) continue;
#pragma unroll
                    for (int u = 0; u < 8; ++u) a += wr[8 * w + u] * vv[w][u];
                }
            } else {
                for (int j = 0; j < TK_KEYS; ++j)
                    if (pg[j] >= 0) a += wr[j] * load_f32(vc + (((size_t)pg[j] * G + c) * pad + d) * P + po[j]);
            }
            acc[e] = a;
        }
    }
    __syncthreads();
    if (S > 1) {
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const int i = owned(e);
            if (i >= n_out) continue;
            const int h = i / p.vdim, d = i % p.vdim;
            p.part_o[(((size_t)row * H + h) * S + split) * p.vdim + d] = acc[e];
        }
        for (int h = tid; h < H; h += 256) {
            const size_t part = ((size_t)row * H + h) * S + split;
            p.part_ml[part * 2] = run_m[h]; p.part_ml[part * 2 + 1] = run_l[h];
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const int i = owned(e);
        if (i >= n_out) continue;
        const float l = run_l[i / p.vdim];
        float v = l > 0.f ? acc[e] / l : 0.f;
        if (p.gate) v *= 1.0f / (1.0f + expf(-p.gate[(size_t)row * p.ldg + i]));
        store_f32(out + i, v);
    }
}

// The blocks along a row's keys leave o_s = sum_j exp(s_j - m_s) v_j, m_s and l_s; with m = max m_s the row's result is
// sum_s exp(m_s - m) o_s / sum_s exp(m_s - m) l_s, times sigmoid(gate).  A block a (row, head).
template <typename T>
__global__ void __launch_bounds__(128)
talking_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, const float* __restrict__ gate, int ldg,
                     T* __restrict__ out, int heads, int vdim, int splits) {
    const size_t row = blockIdx.x;
    const int h = blockIdx.y;
    const size_t base = (row * heads + h) * splits;
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, part_ml[(base + s) * 2]);
    for (int c = threadIdx.x; c < vdim; c += 128) {
        float num = 0.f, den = 0.f;
        for (int s = 0; s < splits; ++s) {
            const float ms = part_ml[(base + s) * 2];
            if (ms == -INFINITY) continue;                       // (a block that saw no key of this row)
            const float w = expf(ms - m);
            num += w * part_o[(base + s) * vdim + c];
            den += w * part_ml[(base + s) * 2 + 1];
        }
        float v = den > 0.f ? num / den : 0.f;
        if (gate) v *= 1.0f / (1.0f + expf(-gate[row * ldg + h * vdim + c]));
        store_f32(out + row * heads * vdim + h * vdim + c, v);
    }
}

static size_t talking_lds(int heads, int pad) {
    return ((size_t)heads * pad + (size_t)heads * heads + 2 * (size_t)heads * TK_KEYS + 3 * (size_t)heads) * sizeof(float) + 2 * TK_KEYS * sizeof(int);
}

template <typename T>
static int launch_talking(const TalkArgs& a, int rows, hipStream_t stream) {
    const size_t lds = talking_lds(a.heads, a.pad);
    const int per = (a.heads * a.vdim + 255) / 256;
    const dim3 grid(rows, a.splits);
    if (lds > 48 * 1024) {                                       // (many heads: the limit of dynamic LDS above the default, once a kernel)
        static bool raised = false;
        if (!raised) {
            const void* kernels[] = {(const void*)attn_talking_kernel<T, 2>, (const void*)attn_talking_kernel<T, 4>, (const void*)attn_talking_kernel<T, 8>,
                                     (const void*)attn_talking_kernel<T, 16>, (const void*)attn_talking_kernel<T, 32>};
            for (const void* k : kernels) {
                const int err = (int)hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
                if (err) return err;
            }
            raised = true;
        }
    }
#define TALK(E) attn_talking_kernel<T, E><<<grid, 256, lds, stream>>>(a)
    if (per <= 2) TALK(2);
    else if (per <= 4) TALK(4);
    else if (per <= 8) TALK(8);
    else if (per <= 16) TALK(16);
    else if (per <= 32) TALK(32);
    else return (int)hipErrorInvalidValue;
#undef TALK
    const int err = CISR_LAUNCH_CHECK();
    if (err || a.splits == 1) return err;
    talking_merge_kernel<T><<<dim3(rows, a.heads), 128, 0, stream>>>(a.part_o, a.part_ml, a.gate, a.ldg, (T*)a.out, a.heads, a.vdim, a.splits);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_attn_talking(const void* q, int q_row_stride, const void* kcache, const void* vcache, const int* tables,
                                 const int* seg_of_row, const int* positions, const float* mix, const float* temp, const float* sink,
                                 const float* gate, int ldg, void* out, int rows, int heads, int kv_heads, int vdim, int pad,
                                 int page_size, int width, int window, int chunk, float scale, int splits, float* part_o, float* part_ml,
                                 int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (splits < 1 || splits > 65535 || heads > 65535 || (splits > 1 && (!part_o || !part_ml))) return (int)hipErrorInvalidValue;
    if (heads <= 0 || kv_heads <= 0 || heads % kv_heads || pad <= 0 || pad % 8 || vdim <= 0 || vdim > pad || page_size <= 0 ||
        !mix || talking_lds(heads, pad) > 160 * 1024 || q_row_stride < heads * pad || (gate && ldg < heads * vdim))
        return (int)hipErrorInvalidValue;
    const TalkArgs a = {q, q_row_stride, kcache, vcache, tables, seg_of_row, positions, mix, temp, sink, gate, ldg, out,
                        heads, kv_heads, vdim, pad, page_size, width, window, chunk, scale, splits, part_o, part_ml};
    return dtype == DT_F32 ? launch_talking<float>(a, rows, stream) : launch_talking<bf16_t>(a, rows, stream);
}
