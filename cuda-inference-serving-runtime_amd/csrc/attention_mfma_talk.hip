// Attention whose scores are mixed over the heads before the softmax, on the matrix cores: prompt portions and mixed
// steps in bfloat16.  (csrc/attention_talking.hip states the law and is the exact float form: single tokens, float32.)
//
// A block owns a tile of up to 16 consecutive rows of one segment (a task list gives segment, first row, rows) and ALL
// query heads of those rows, because a (row, key) pair's mixed score needs every head's raw score.  Wave w owns the
// heads w HPW .. w HPW + HPW - 1.  Keys are walked 32 at a time, tiles at absolute multiples of 32:
//   (A) raw scores S_g = Q_g K^T of the wave's heads, `v_mfma_f32_16x16x32_bf16`, queries and keys loaded 16 bytes a
//       lane straight from memory into operands; the 16 x 32 float scores of a head go to LDS
//   (B) a thread a (row, key) pair: all heads' raw scores from LDS, the mix s_h = sum_g mix[h, g] temp[g] scale raw_g in
//       float, keys that the row does not see (its block of positions, its own position) set to minus infinity, back
//       into LDS in place
//   (C) two lanes a (head, row): running maximum and denominator over the tile's 32 keys, weights exp(s - m) as bf16
//       into LDS, the factor that rescales what was summed before
//   (D) O_h += P_h V of the wave's heads on the matrix cores: weights from LDS, eight keys of a transposed value page a
//       16-byte load (asked for at the head of the step where a wave has at most two heads: the loads fly while the
//       scores are made); keys past the tile's last row are cleared on the way (a fresh page may hold anything)
// Three barriers a tile.  Where a step has too few tiles to fill the GPU, `splits` blocks share a tile's keys (block s
// walks the steps s, s + splits, ...) and a small kernel merges their sums.  The sink is a key of score sink_h and no value: it starts the running maximum and the
// denominator.  Pages hold heads of `pad` coordinates (a multiple of 8, at most 32 PT) whose rest is zero; pages of a
// multiple of 8 keys.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define TT_ROWS 16
#define TT_KEYS 32
#define TT_RS 33          // floats a row of scores takes in LDS (33: rows a bank apart)
#define TT_PS 40          // bf16 a row of weights takes in LDS (80 bytes: the 16 rows' 16-byte reads fall into different banks)
#define TT_MAX_HEADS 32

struct TalkTileArgs {
    const bf16_t* q; int q_row_stride;
    const bf16_t* kcache; const bf16_t* vcache;
    const int* tables; const int* tasks; const int* positions;
    const float* mix; const float* temp; const float* sink;
    const float* gate; int ldg;
    bf16_t* out;
    int heads, kv_heads, vdim, pad, page_size, width, window, chunk;
    float scale;
    int splits; float* part_o; float* part_ml;      // splits > 1: block (tile, s) walks the steps s, s + splits, ... and leaves sums
};

template <int HPW, int PT>
__global__ void __launch_bounds__(512)
attn_talking_tiles_kernel(TalkTileArgs p) {
    extern __shared__ float lds[];
    const int H = p.heads, G = p.kv_heads, pad = p.pad, P = p.page_size, group = H / G;
    const int NT = blockDim.x;
    float* sraw = lds;                                    // [H, 16, TT_RS]
    constexpr int HMAX = 8 * HPW;                         // heads a block of this build takes at most
    float* mixw = sraw + H * TT_ROWS * TT_RS;             // [H, HMAX]: mix[h, g] temp[g] scale, zero from column H on
    float* run_m = mixw + H * HMAX;                       // [H, 16]
    float* run_l = run_m + H * TT_ROWS;
    float* alpha = run_l + H * TT_ROWS;
    int* lo = (int*)(alpha + H * TT_ROWS);                // [16]: first key a row sees
    int* hi = lo + TT_ROWS;                               // [16]: one past the last (0: the tile has no such row)
    bf16_t* pw = (bf16_t*)(hi + TT_ROWS);                 // [H, 16, TT_PS]

    const int tid = threadIdx.x, lane = tid % WAVE, wave = tid / WAVE;
    const int r = lane % 16, g8 = lane / 16;
    const int seg = p.tasks[blockIdx.x * 4];
    if (seg < 0) return;
    const int first = p.tasks[blockIdx.x * 4 + 1], n_rows = p.tasks[blockIdx.x * 4 + 2];
    if (tid < TT_ROWS) {
        int a = 0, b = 0;
        if (tid < n_rows) {
            const int pos = p.positions[first + tid];
            b = pos + 1;
            a = p.chunk > 0 ? (pos / p.chunk) * p.chunk : (p.window > 0 && b > p.window) ? b - p.window : 0;
        }
        lo[tid] = a; hi[tid] = b;
    }
    for (int i = tid; i < H * HMAX; i += NT) {
        const int h = i / HMAX, g = i % HMAX;
        mixw[i] = g < H ? p.mix[h * H + g] * (p.temp ? p.temp[g] : 1.0f) * p.scale : 0.f;
    }
    const int split = blockIdx.y, S = p.splits;
    for (int i = tid; i < H * TT_ROWS; i += NT) {
        const bool sunk = p.sink && split == 0;               // (the sink counts once: in the first block along the keys)
        run_m[i] = sunk ? p.sink[i / TT_ROWS] : -INFINITY;
        run_l[i] = sunk ? 1.0f : 0.f;
    }
    __syncthreads();
    const int begin = lo[0], end = hi[n_rows - 1];        // (positions ascend: the first row sees furthest back)
    const int* table = p.tables + (size_t)seg * p.width;
    const int h0 = wave * HPW;
    f32x4 o[HPW][2 * PT];
#pragma unroll
    for (int i = 0; i < HPW; ++i)
#pragma unroll
        for (int t = 0; t < 2 * PT; ++t) o[i][t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    const u32x4 zero = {0u, 0u, 0u, 0u};
    const bf16_t* qrow = p.q + (size_t)(first + min(r, n_rows - 1)) * p.q_row_stride;

    constexpr bool AHEAD = HPW <= 2;                             // the step's values are asked for before its scores are made
    // the pages of this lane's keys (scores: key r of either half of the tile; values: eight keys from g8 * 8), asked
    // for a step ahead: a step's loads of keys and values then leave at its head
    int kpage[2], vpage, kpage_next[2], vpage_next;
    auto pages_of = [&](int base, int (&kp)[2], int& vp) {
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            const int t = base + sub * 16 + r;
            kp[sub] = (t >= begin && t < end) ? table[t / P] : -1;
        }
        const int tv = base + g8 * 8;
        vp = (tv < end && tv + 8 > begin) ? table[tv / P] : -1;
    };
    const int base0 = begin / TT_KEYS * TT_KEYS + split * TT_KEYS;
    pages_of(base0, kpage_next, vpage_next);
    for (int base = base0; base < end; base += S * TT_KEYS) {
        kpage[0] = kpage_next[0]; kpage[1] = kpage_next[1]; vpage = vpage_next;
        pages_of(base + S * TT_KEYS, kpage_next, vpage_next);
        const int tv = base + g8 * 8;
        const int live = end - tv;                               // keys of the eight that are written (>= 8: all)
        auto values = [&](int c, int vt) {
            const int cc = vt * 16 + r;
            u32x4 vf = zero;
            if (vpage >= 0 && cc < p.vdim) {
                vf = *(const u32x4*)(p.vcache + (((size_t)vpage * G + c) * pad + cc) * P + tv % P);
                if (live < 8) {                                  // clear what lies past the last key of the tile's rows
                    uint32_t w[4] = {vf.x, vf.y, vf.z, vf.w};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (2 * e >= live) w[e] = 0u;
                        else if (2 * e + 1 >= live) w[e] &= 0xffffu;
                    }
                    vf = (u32x4){w[0], w[1], w[2], w[3]};
                }
            }
            return vf;
        };
        u32x4 vahead[AHEAD ? HPW : 1][2 * PT];
        if (AHEAD) {
#pragma unroll
            for (int i = 0; i < HPW; ++i)
#pragma unroll
                for (int vt = 0; vt < 2 * PT; ++vt)
                    vahead[i][vt] = (h0 + i < H && vt * 16 < p.vdim) ? values((h0 + i) / group, vt) : zero;
        }
        // ---- (A) raw scores of this wave's heads: all of a head's loads on their way before its matrix instructions
        u32x4 kf[2][PT];
        int c_loaded = -1;                                       // the key head whose keys kf holds (heads of one group share them)
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int h = h0 + i;
            if (h >= H) continue;
            const int c = h / group;
            u32x4 qf[PT];
#pragma unroll
            for (int ks = 0; ks < PT; ++ks) {
                const int d = ks * 32 + g8 * 8;
                qf[ks] = (d < pad && r < n_rows) ? *(const u32x4*)(qrow + (size_t)h * pad + d) : zero;
            }
            if (c != c_loaded) {
                c_loaded = c;
#pragma unroll
                for (int ks = 0; ks < PT; ++ks) {
                    const int d = ks * 32 + g8 * 8;
#pragma unroll
                    for (int sub = 0; sub < 2; ++sub) {
                        const int t = base + sub * 16 + r;
                        const bf16_t* kr = p.kcache + (((size_t)max(kpage[sub], 0) * G + c) * P + t % P) * pad;
                        kf[sub][ks] = (kpage[sub] >= 0 && d < pad) ? *(const u32x4*)(kr + d) : zero;
                    }
                }
            }
#pragma unroll
            for (int sub = 0; sub < 2; ++sub) {
                f32x4 st = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < PT; ++ks)
                    st = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, qf[ks]), __builtin_bit_cast(bf16x8, kf[sub][ks]), st, 0, 0, 0);
#pragma unroll
                for (int x = 0; x < 4; ++x) sraw[(h * TT_ROWS + g8 * 4 + x) * TT_RS + sub * 16 + r] = st[x];
            }
        }
        __syncthreads();
        // ---- (B) the mix over the heads, a thread a (row, key) pair
        for (int pair = tid; pair < TT_ROWS * TT_KEYS; pair += NT) {
            const int row = pair / TT_KEYS, key = pair % TT_KEYS, t = base + key;
            const bool seen = t >= lo[row] && t < hi[row];
            float v[HMAX];
#pragma unroll
            for (int g = 0; g < HMAX; ++g) v[g] = g < H ? sraw[(g * TT_ROWS + row) * TT_RS + key] : 0.f;
            for (int h = 0; h < H; ++h) {
                const float4* mw = (const float4*)(mixw + h * HMAX);          // (columns past H are zero: no test in the sum)
                float s = 0.f;
#pragma unroll
                for (int g = 0; g < HMAX; g += 4) {
                    const float4 m4 = mw[g / 4];
                    s += m4.x * v[g] + m4.y * v[g + 1] + m4.z * v[g + 2] + m4.w * v[g + 3];
                }
                sraw[(h * TT_ROWS + row) * TT_RS + key] = seen ? s : -INFINITY;
            }
        }
        __syncthreads();
        // ---- (C) running maximum, denominator and weights: two neighbouring lanes a (head, row), 16 keys each
        for (int it = tid; it < 2 * H * TT_ROWS; it += NT) {
            const int item = it / 2, half = it % 2;
            const float* sr = sraw + item * TT_RS + half * 16;
            float mx = -INFINITY;
#pragma unroll
            for (int k = 0; k < 16; ++k) mx = fmaxf(mx, sr[k]);
            mx = fmaxf(mx, __shfl_xor(mx, 1, WAVE));
            const float m_old = run_m[item], m_new = fmaxf(m_old, mx);
            const bool none = m_new == -INFINITY;              // nothing seen so far and no sink
            const float a = none ? 1.0f : expf(m_old - m_new);
            float sum = 0.f;
            bf16_t* wr = pw + item * TT_PS + half * 16;
#pragma unroll
            for (int k = 0; k < 16; k += 2) {
                const float w0 = none ? 0.f : expf(sr[k] - m_new), w1 = none ? 0.f : expf(sr[k + 1] - m_new);
                sum += w0 + w1;
                *(uint32_t*)(wr + k) = pack_bf16x2(w0, w1);
            }
            sum += __shfl_xor(sum, 1, WAVE);
            if (half == 0) {
                run_m[item] = m_new;
                run_l[item] = run_l[item] * a + sum;
                alpha[item] = a;
            }
        }
        __syncthreads();
        // ---- (D) the values of this wave's heads
#pragma unroll
        for (int i = 0; i < HPW; ++i) {
            const int h = h0 + i;
            if (h >= H) continue;
            const int c = h / group;
            float al[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) al[x] = alpha[h * TT_ROWS + g8 * 4 + x];
            const bf16x8 pf = *(const bf16x8*)(pw + (h * TT_ROWS + r) * TT_PS + g8 * 8);
#pragma unroll
            for (int vt = 0; vt < 2 * PT; ++vt) {
                if (vt * 16 >= p.vdim) continue;
                const u32x4 vf = AHEAD ? vahead[AHEAD ? i : 0][vt] : values(c, vt);
#pragma unroll
                for (int x = 0; x < 4; ++x) o[i][vt][x] *= al[x];
                o[i][vt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, __builtin_bit_cast(bf16x8, vf), o[i][vt], 0, 0, 0);
            }
        }
        // (the next tile's (A) writes only the scores, which nobody reads after the barrier before (D))
    }
    __syncthreads();
    const int n_out = H * p.vdim;
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
        const int h = h0 + i;
        if (h >= H) continue;
#pragma unroll
        for (int vt = 0; vt < 2 * PT; ++vt) {
            const int cc = vt * 16 + r;
            if (cc >= p.vdim) continue;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                const int row = g8 * 4 + x;
                if (row >= n_rows) continue;
                if (S > 1) {                                     // sums for the merge: what this block's keys add up to
                    const size_t part = ((size_t)(first + row) * H + h) * S + split;
                    p.part_o[part * p.vdim + cc] = o[i][vt][x];
                    if (vt == 0 && r == 0) { p.part_ml[part * 2] = run_m[h * TT_ROWS + row]; p.part_ml[part * 2 + 1] = run_l[h * TT_ROWS + row]; }
                    continue;
                }
                const float l = run_l[h * TT_ROWS + row];
                float v = l > 0.f ? o[i][vt][x] / l : 0.f;
                const size_t at = (size_t)(first + row);
                if (p.gate) v *= 1.0f / (1.0f + expf(-p.gate[at * p.ldg + h * p.vdim + cc]));
                p.out[at * n_out + h * p.vdim + cc] = f32_to_bf16(v);
            }
        }
    }
}

// The blocks along a tile's keys leave o_s = sum_j exp(s_j - m_s) v_j, m_s and l_s = sum_j exp(s_j - m_s); with m = max m_s the
// row's result is sum_s exp(m_s - m) o_s / sum_s exp(m_s - m) l_s, times sigmoid(gate).  A block a (row, head).
__global__ void __launch_bounds__(128)
talk_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, const float* __restrict__ gate, int ldg,
                  bf16_t* __restrict__ out, int heads, int vdim, int splits) {
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
        out[row * heads * vdim + h * vdim + c] = f32_to_bf16(v);
    }
}

static size_t talk_tiles_lds(int heads) {
    const int hmax = heads <= 8 ? 8 : heads <= 16 ? 16 : 32;
    return ((size_t)heads * TT_ROWS * TT_RS + (size_t)heads * hmax + 3 * (size_t)heads * TT_ROWS) * sizeof(float) + 2 * TT_ROWS * sizeof(int) +
           (size_t)heads * TT_ROWS * TT_PS * sizeof(bf16_t);
}

// Whether the tile kernel takes these sizes: up to 32 heads, heads of up to 128 coordinates, pages of a multiple of 8 keys.
extern "C" int cisr_attn_talking_tiles_ok(int heads, int kv_heads, int vdim, int pad, int page_size) {
    return heads > 0 && heads <= TT_MAX_HEADS && kv_heads > 0 && heads % kv_heads == 0 && pad > 0 && pad % 8 == 0 && pad <= 128 &&
           vdim > 0 && vdim <= pad && page_size > 0 && page_size % 8 == 0 && talk_tiles_lds(heads) <= 160 * 1024;
}

template <int HPW, int PT>
static int launch_tiles(const TalkTileArgs& a, int tiles, hipStream_t stream) {
    const dim3 grid(tiles, a.splits);
    const size_t lds = talk_tiles_lds(a.heads);
    const int waves = (a.heads + HPW - 1) / HPW;
    if (lds > 48 * 1024) {
        static bool raised = false;                              // (once a kernel: the limit of dynamic LDS above the default)
        if (!raised) {
            const int err = (int)hipFuncSetAttribute((const void*)attn_talking_tiles_kernel<HPW, PT>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
            if (err) return err;
            raised = true;
        }
    }
    attn_talking_tiles_kernel<HPW, PT><<<grid, waves * WAVE, lds, stream>>>(a);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_attn_talking_tiles(const void* q, int q_row_stride, const void* kcache, const void* vcache, const int* tables,
                                       const int* tasks, int tiles, const int* positions, const float* mix, const float* temp,
                                       const float* sink, const float* gate, int ldg, void* out, int heads, int kv_heads, int vdim,
                                       int pad, int page_size, int width, int window, int chunk, float scale, int rows, int splits,
                                       float* part_o, float* part_ml, hipStream_t stream) {
    if (tiles <= 0) return 0;
    if (splits < 1 || splits > 64 || (splits > 1 && (!part_o || !part_ml || rows <= 0))) return (int)hipErrorInvalidValue;
    if (!cisr_attn_talking_tiles_ok(heads, kv_heads, vdim, pad, page_size) || !mix || q_row_stride < heads * pad || q_row_stride % 8 ||
        (gate && ldg < heads * vdim))
        return (int)hipErrorInvalidValue;
    const TalkTileArgs a = {(const bf16_t*)q, q_row_stride, (const bf16_t*)kcache, (const bf16_t*)vcache, tables, tasks, positions, mix, temp,
                            sink, gate, ldg, (bf16_t*)out, heads, kv_heads, vdim, pad, page_size, width, window, chunk, scale, splits, part_o, part_ml};
    const int hpw = heads <= 8 ? 1 : heads <= 16 ? 2 : 4;
    const int pt = (pad + 31) / 32;
#define TILES(HPW) (pt == 1 ? launch_tiles<HPW, 1>(a, tiles, stream) : pt == 2 ? launch_tiles<HPW, 2>(a, tiles, stream) : \
                    pt == 3 ? launch_tiles<HPW, 3>(a, tiles, stream) : launch_tiles<HPW, 4>(a, tiles, stream))
    const int err = hpw == 1 ? TILES(1) : hpw == 2 ? TILES(2) : TILES(4);
#undef TILES
    if (err || splits == 1) return err;
    talk_merge_kernel<<<dim3(rows, heads), 128, 0, stream>>>(part_o, part_ml, gate, ldg, (bf16_t*)out, heads, vdim, splits);
    return CISR_LAUNCH_CHECK();
}
