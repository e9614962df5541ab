// Routed experts: each row of a step goes through the `top` experts with the largest router logits.
//
//   route      logits float [T, E] (+ bias) -> the chosen experts [T, top] (largest first, the lowest index wins a tie)
//              and their weights, the softmax over the chosen logits only, float
//   arrange    the T top (row, choice) pairs ordered by expert, every expert's run padded to a whole number of 64-row
//              tiles: pair_of_pos[pos] (-1: padding) and tile_expert[tile] (-1: no tile).  One block; the order of
//              pairs inside an expert's run is whatever the atomics give, which no result depends on (a pair's
//              arithmetic does not know its place).
//   products   per tile of 64 pairs one expert's matrix: up  = act(h[row of pair] . Wup[e]^T) stored by place,
//              down = up[place] . Wdown[e]^T stored by pair, float [T top, H]; the weighted sum over a row's pairs
//              is left to the kernel that reads them next.
// bf16 operands run on the matrix cores (K a multiple of 8, 16-byte aligned rows); everything else, and the true
// 32-bit path, runs the plain FMA kernel with float accumulation in ascending k order.
#include "common.h"

#define EX_TILE 64
#define MAX_TOP 16

__global__ void __launch_bounds__(256)
route_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ bias, int* __restrict__ chosen,
             float* __restrict__ weights, int rows, int experts, int top) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= rows) return;
    const float* lr = logits + (size_t)row * ld;
    int ids[MAX_TOP];
    float vals[MAX_TOP];
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = -INFINITY;
        for (int e = 0; e < experts; ++e) {
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= ids[j] == e;
            if (taken) continue;
            const float v = lr[e] + (bias ? bias[e] : 0.f);
            if (best < 0 || v > bv) { best = e; bv = v; }
        }
        ids[k] = best;
        vals[k] = bv;
    }
    float den = 0.f;
    const float largest = vals[0];
    for (int k = 0; k < top; ++k) { vals[k] = expf(vals[k] - largest); den += vals[k]; }
    for (int k = 0; k < top; ++k) {
        chosen[(size_t)row * top + k] = ids[k];
        weights[(size_t)row * top + k] = vals[k] / den;
    }
}

__global__ void __launch_bounds__(1024)
arrange_kernel(const int* __restrict__ chosen, int pairs, int experts, int max_tiles, int* __restrict__ pair_of_pos,
               int* __restrict__ tile_expert) {
    extern __shared__ int lds[];          // counts[E], then start[E] (in places), then cursor[E]
    int* counts = lds;
    int* start = lds + experts;
    int* cursor = lds + 2 * experts;
    for (int e = threadIdx.x; e < experts; e += 1024) counts[e] = 0;
    for (int p = threadIdx.x; p < max_tiles * EX_TILE; p += 1024) pair_of_pos[p] = -1;
    for (int t = threadIdx.x; t < max_tiles; t += 1024) tile_expert[t] = -1;
    __syncthreads();
    for (int p = threadIdx.x; p < pairs; p += 1024) {
        const int e = chosen[p];
        if (e >= 0 && e < experts) atomicAdd(&counts[e], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int at = 0;
        for (int e = 0; e < experts; ++e) {
            start[e] = cursor[e] = at;
            at += (counts[e] + EX_TILE - 1) / EX_TILE * EX_TILE;
        }
    }
    __syncthreads();
    for (int e = threadIdx.x; e < experts; e += 1024) {
        const int first = start[e] / EX_TILE, n = (counts[e] + EX_TILE - 1) / EX_TILE;
        for (int t = 0; t < n; ++t) if (first + t < max_tiles) tile_expert[first + t] = e;
    }
    for (int p = threadIdx.x; p < pairs; p += 1024) {
        const int e = chosen[p];
        if (e < 0 || e >= experts) continue;
        const int pos = atomicAdd(&cursor[e], 1);
        if (pos < max_tiles * EX_TILE) pair_of_pos[pos] = p;
    }
}

extern "C" int cisr_experts_route(const float* logits, int ld, const float* bias, int* chosen, float* weights, int rows,
                                  int experts, int top, int max_tiles, int* pair_of_pos, int* tile_expert, hipStream_t stream) {
    if (rows <= 0) return 0;
    const bool arrange = pair_of_pos != nullptr;        // (null: the caller wants the choice only)
    if (experts <= 0 || top <= 0 || top > MAX_TOP || top > experts || experts > 4096 || (arrange && (!tile_expert ||
        (long long)max_tiles * EX_TILE < (long long)rows * top + (long long)experts * (EX_TILE - 1))))
        return (int)hipErrorInvalidValue;
    route_kernel<<<(rows + 255) / 256, 256, 0, stream>>>(logits, ld, bias, chosen, weights, rows, experts, top);
    int err = CISR_LAUNCH_CHECK();
    if (err || !arrange) return err;
    arrange_kernel<<<1, 1024, 3 * experts * sizeof(int), stream>>>(chosen, rows * top, experts, max_tiles, pair_of_pos, tile_expert);
    return CISR_LAUNCH_CHECK();
}

// Routing by scores: s = softmax of the logits over all `outputs` of the router; the choice goes by s + correction
// (null: by s), held to the `keep` groups, of `groups` equal groups of neighbours, whose largest choice score is
// largest (groups 0: no groups); the `top` largest are chosen (the lowest index wins a tie) and weigh s itself, not
// normed again.  A thread a row; float arithmetic.
__global__ void __launch_bounds__(256)
route_scored_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction, int* __restrict__ chosen,
                    float* __restrict__ weights, int rows, int outputs, int top, int groups, int keep) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    if (row >= rows) return;
    const float* lr = logits + (size_t)row * ld;
    float largest = -INFINITY, den = 0.f;
    for (int e = 0; e < outputs; ++e) largest = fmaxf(largest, lr[e]);
    for (int e = 0; e < outputs; ++e) den += expf(lr[e] - largest);
    auto score = [&](int e) { return expf(lr[e] - largest) / den; };
    auto choice = [&](int e) { return score(e) + (correction ? correction[e] : 0.f); };
    unsigned long long kept = ~0ull;                       // groups that may be chosen from (at most 64 groups)
    const int per = groups > 0 ? outputs / groups : outputs;
    if (groups > 0) {
        kept = 0ull;
        for (int k = 0; k < keep; ++k) {
            int best = -1;
            float bv = -INFINITY;
            for (int g = 0; g < groups; ++g) {
                if ((kept >> g) & 1ull) continue;
                float gv = -INFINITY;
                for (int e = g * per; e < (g + 1) * per; ++e) gv = fmaxf(gv, choice(e));
                if (best < 0 || gv > bv) { best = g; bv = gv; }
            }
            kept |= 1ull << best;
        }
    }
    int ids[MAX_TOP];
    for (int k = 0; k < top; ++k) {
        int best = -1;
        float bv = -INFINITY;
        for (int e = 0; e < outputs; ++e) {
            if (groups > 0 && !((kept >> (e / per)) & 1ull)) continue;
            bool taken = false;
            for (int j = 0; j < k; ++j) taken |= ids[j] == e;
            if (taken) continue;
            const float v = choice(e);
            if (best < 0 || v > bv) { best = e; bv = v; }
        }
        ids[k] = best;
        chosen[(size_t)row * top + k] = best;
        weights[(size_t)row * top + k] = score(best);
    }
}

// The same routing with a wave a row (routers of at most 512 outputs): lane l holds the outputs l, l + 64, ...; the
// maximum, the sum, a group's best and every choice are reductions over the wave, so a step of few rows does not wait
// for one thread's chain of exponentials.  The lowest index wins a tie, as above.
#define ROUTE_PER_LANE 8
__global__ void __launch_bounds__(256)
route_scored_wave_kernel(const float* __restrict__ logits, int ld, const float* __restrict__ correction, int* __restrict__ chosen,
                         float* __restrict__ weights, int rows, int outputs, int top, int groups, int keep) {
    const int row = blockIdx.x * 4 + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (row >= rows) return;
    const float* lr = logits + (size_t)row * ld;
    float z[ROUTE_PER_LANE], largest = -INFINITY;
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + WAVE * i;
        z[i] = e < outputs ? lr[e] : -INFINITY;
        largest = fmaxf(largest, z[i]);
    }
    largest = wave_max(largest);
    float den = 0.f, s[ROUTE_PER_LANE], c[ROUTE_PER_LANE];
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) { s[i] = lane + WAVE * i < outputs ? expf(z[i] - largest) : 0.f; den += s[i]; }
    den = wave_sum(den);
#pragma unroll
    for (int i = 0; i < ROUTE_PER_LANE; ++i) {
        const int e = lane + WAVE * i;
        s[i] /= den;
        c[i] = e < outputs ? s[i] + (correction ? correction[e] : 0.f) : -INFINITY;      // -inf: not there, dropped or taken
    }
    // the best (value, lowest index) over the wave among this lane's candidates `v`
    auto best_of = [&](const float (&v)[ROUTE_PER_LANE], float& bv, int& be) {
        bv = -INFINITY; be = 0x7fffffff;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            const int e = lane + WAVE * i;
            if (e < outputs && (v[i] > bv || (v[i] == bv && e < be))) { bv = v[i]; be = e; }
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, WAVE);
            const int oe = __shfl_xor(be, off, WAVE);
            if (ov > bv || (ov == bv && oe < be)) { bv = ov; be = oe; }
        }
    };
    if (groups > 0) {
        const int per = outputs / groups;
        unsigned long long kept = 0ull;
        for (int k = 0; k < keep; ++k) {
            // the group, not kept yet, whose largest choice score is largest (the lowest group wins a tie): a group's
            // largest score is the score of its best member, and of two equal ones the lower index lies in the lower group
            float v[ROUTE_PER_LANE];
#pragma unroll
            for (int i = 0; i < ROUTE_PER_LANE; ++i) {
                const int e = lane + WAVE * i;
                v[i] = (e < outputs && !((kept >> (e / per)) & 1ull)) ? c[i] : -INFINITY;
            }
            float bv; int be;
            best_of(v, bv, be);
            int g = be / per;
            if (bv == -INFINITY) {                               // (every candidate at minus infinity: the lowest group not kept)
                g = 0;
                while ((kept >> g) & 1ull) ++g;
            }
            kept |= 1ull << g;
        }
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            const int e = lane + WAVE * i;
            if (e < outputs && !((kept >> (e / per)) & 1ull)) c[i] = -INFINITY;
        }
    }
    for (int k = 0; k < top; ++k) {
        float bv; int be;
        best_of(c, bv, be);
        float share = 0.f;
#pragma unroll
        for (int i = 0; i < ROUTE_PER_LANE; ++i) {
            if (lane + WAVE * i == be) { share = s[i]; c[i] = -INFINITY; }
        }
        share = wave_sum(share);                                 // (one lane holds it)
        if (lane == 0) { chosen[(size_t)row * top + k] = be; weights[(size_t)row * top + k] = share; }
    }
}

// `experts` of the router's `outputs` have matrices (the first ones): only their pairs are arranged into tiles.
extern "C" int cisr_experts_route_scored(const float* logits, int ld, const float* correction, int* chosen, float* weights, int rows,
                                         int outputs, int experts, int top, int groups, int keep, int max_tiles, int* pair_of_pos,
                                         int* tile_expert, hipStream_t stream) {
    if (rows <= 0) return 0;
    const bool arrange = pair_of_pos != nullptr;
    if (outputs <= 0 || experts <= 0 || experts > outputs || top <= 0 || top > MAX_TOP || top > outputs || experts > 4096 || groups < 0 ||
        groups > 64 || (groups > 0 && (outputs % groups || keep <= 0 || keep > groups || keep * (outputs / groups) < top)) ||
        (arrange && (!tile_expert || (long long)max_tiles * EX_TILE < (long long)rows * top + (long long)experts * (EX_TILE - 1))))
        return (int)hipErrorInvalidValue;
    // steps of few rows: a wave a row; many rows keep a thread a row (the GPU is full either way, and a thread's chain is short beside the step)
    if (outputs <= WAVE * ROUTE_PER_LANE && rows <= 4096)
        route_scored_wave_kernel<<<(rows + 3) / 4, 256, 0, stream>>>(logits, ld, correction, chosen, weights, rows, outputs, top, groups, keep);
    else
        route_scored_kernel<<<(rows + 255) / 256, 256, 0, stream>>>(logits, ld, correction, chosen, weights, rows, outputs, top, groups, keep);
    int err = CISR_LAUNCH_CHECK();
    if (err || !arrange) return err;
    arrange_kernel<<<1, 1024, 3 * experts * sizeof(int), stream>>>(chosen, rows * top, experts, max_tiles, pair_of_pos, tile_expert);
    return CISR_LAUNCH_CHECK();
}

// y[row] = sum_k weights[row, k] * (chosen[row, k] < experts ? down[row top + k] : x[row]) + shared[row]: the weighted sum
// over a row's choices, a choice without matrices being the sublayer's input itself (x, in the activations' type), plus
// what every row goes through.
template <typename TX>
__global__ void __launch_bounds__(256)
experts_combine_kernel(const float* __restrict__ down, const float* __restrict__ weights, const int* __restrict__ chosen,
                       const TX* __restrict__ x, const float* __restrict__ shared, float* __restrict__ y, int dim, int top,
                       int experts) {
    const size_t row = blockIdx.x;
    float w[MAX_TOP];
    int real[MAX_TOP];
    for (int k = 0; k < top; ++k) {
        w[k] = weights[row * top + k];
        const int e = chosen[row * top + k];
        real[k] = e >= 0 && e < experts;
    }
    for (int d = threadIdx.x; d < dim; d += 256) {
        float v = shared ? shared[row * dim + d] : 0.f;
        for (int k = 0; k < top; ++k) v += w[k] * (real[k] ? down[(row * top + k) * dim + d] : load_f32(x + row * dim + d));
        y[row * dim + d] = v;
    }
}

extern "C" int cisr_experts_combine(const float* down, const float* weights, const int* chosen, const void* x, int x_dtype,
                                    const float* shared, float* y, int rows, int dim, int top, int experts, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (dim <= 0 || top <= 0 || top > MAX_TOP || experts < 0) return (int)hipErrorInvalidValue;
    if (x_dtype == DT_F32) experts_combine_kernel<float><<<rows, 256, 0, stream>>>(down, weights, chosen, (const float*)x, shared, y, dim, top, experts);
    else experts_combine_kernel<bf16_t><<<rows, 256, 0, stream>>>(down, weights, chosen, (const bf16_t*)x, shared, y, dim, top, experts);
    return CISR_LAUNCH_CHECK();
}

// relu(z)^2, the experts' activation; ACT 0: none
template <int ACT>
__device__ __forceinline__ float expert_act(float v) {
    if (ACT == 0) return v;
    const float r = fmaxf(v, 0.f);
    return r * r;
}

// rows of a tile: where the operand's row of a place lies, and where its result goes (-1: padding)
struct TileRows { int a, c; };
__device__ __forceinline__ TileRows tile_rows(int pos, int pair, int gather_div, int scatter) {
    TileRows t;
    t.a = pair < 0 ? -1 : gather_div > 0 ? pair / gather_div : pos;
    t.c = pair < 0 ? -1 : scatter ? pair : pos;
    return t;
}

// ------------------------------------------------------------------ plain FMA tiles (any type, any size)
template <typename TA, typename TC, int ACT>
__global__ void __launch_bounds__(256)
expert_gemm_fma_kernel(const TA* __restrict__ A, int lda, const TA* __restrict__ W, const int* __restrict__ tile_expert,
                       const int* __restrict__ pair_of_pos, int gather_div, int scatter, TC* __restrict__ C, int ldc, int N, int K) {
    const int tile = blockIdx.x;
    const int e = tile_expert[tile];
    if (e < 0) return;
    __shared__ float As[16][EX_TILE + 4];
    __shared__ float Ws[16][EX_TILE + 4];
    __shared__ int arow[EX_TILE], crow[EX_TILE];
    const int tid = threadIdx.x;
    if (tid < EX_TILE) {
        const int pos = tile * EX_TILE + tid;
        const TileRows t = tile_rows(pos, pair_of_pos[pos], gather_div, scatter);
        arow[tid] = t.a; crow[tid] = t.c;
    }
    __syncthreads();
    const int n0 = blockIdx.y * EX_TILE;
    const TA* We = W + (size_t)e * N * K;
    const int ty = tid / 16, tx = tid % 16;
    const int lr = tid / 4, lk = (tid % 4) * 4;
    float acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
    for (int k0 = 0; k0 < K; k0 += 16) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int k = k0 + lk + x;
            const int am = arow[lr], wn = n0 + lr;
            As[lk + x][lr] = (am >= 0 && k < K) ? load_f32(A + (size_t)am * lda + k) : 0.f;
            Ws[lk + x][lr] = (wn < N && k < K) ? load_f32(We + (size_t)wn * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            float a[4], w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tx * 4 + j];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int m = crow[ty * 4 + i];
        if (m < 0) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + tx * 4 + j;
            if (n < N) store_f32(C + (size_t)m * ldc + n, expert_act<ACT>(acc[i][j]));
        }
    }
}

// ------------------------------------------------------------------ matrix-core tiles (bf16, K a multiple of 8)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define EX_BK 64
#define EX_BN 128
#define EX_PAIRED_FROM 48   // tiles a step can take from which a block takes two tiles of one expert at a time
#define EX_LD 72         // bf16 elements a tile row takes in LDS (144 bytes: 16-byte chunks, rows spread over the banks)

// A block of four waves owns 64 MT places x 128 columns; wave (wm, wn) the places 32 MT wm .. 32 MT wm + 32 MT - 1 and
// the columns 64 wn .. 64 wn + 63: 2 MT x 4 tiles of 16 x 16, 16 MT matrix instructions a 64-deep step against 2 MT + 4
// operand reads.  Operands go global memory -> registers -> LDS (two buffers, one barrier a step) -> matrix-core
// operands; the next step's global loads (MT 1: the next two steps') are in flight while this one is multiplied.
// MT 2 (steps of many rows): the block of a tile that is the first, third, ... of its expert's run also takes the tile
// after it if that is the same expert's (else its second half is padding), and the block of the other tile leaves at
// once: every byte of the expert's matrix then meets twice the rows.
template <typename TC, int ACT, int MT>
__global__ void __launch_bounds__(256)
expert_gemm_mfma_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const int* __restrict__ tile_expert,
                        const int* __restrict__ pair_of_pos, int gather_div, int scatter, TC* __restrict__ C, int ldc, int N, int K,
                        int tiles) {
    // The hardware deals consecutive blocks round-robin to the 8 XCDs, each with an L2 of its own.  Renumber so that an
    // XCD gets a contiguous run of (tile, column block) pairs, tiles fastest: the tiles of one expert follow each other,
    // so the blocks that read the same 128 rows of that expert's matrix run on one XCD at about the same time.
    // The grid is one row of blocks, rounded up to a multiple of 8.
    const int blocks = tiles * ((N + EX_BN - 1) / EX_BN);
    const int per_xcd = (blocks + 7) / 8;
    const int slot = ((int)blockIdx.x % 8) * per_xcd + (int)blockIdx.x / 8;
    if (slot >= blocks) return;
    const int tile = slot % tiles, column_block = slot / tiles;
    const int e = tile_expert[tile];
    if (e < 0) return;
    int places = EX_TILE;              // places of this block that are not padding by construction
    if (MT == 2) {
        int before = 0;                // tiles of this expert's run before this one
        while (tile - before - 1 >= 0 && tile_expert[tile - before - 1] == e) ++before;
        if (before & 1) return;
        if (tile + 1 < tiles && tile_expert[tile + 1] == e) places = 2 * EX_TILE;
    }
    __shared__ __attribute__((aligned(16))) bf16_t As[2][MT * EX_TILE * EX_LD];
    __shared__ __attribute__((aligned(16))) bf16_t Ws[2][EX_BN * EX_LD];
    __shared__ int crow[MT * EX_TILE];
    const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / WAVE), lane = tid % WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int r = lane % 16, g = lane / 16;
    const int lr = tid / 8, lc = (tid % 8) * 8;               // this thread's chunks of a tile: rows lr + 32 i, first k
    const int n0 = column_block * EX_BN;
    const bf16_t* ap[2 * MT];
    const bf16_t* wp[4];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
        const int row = lr + 32 * i;
        const int pos = tile * EX_TILE + row;
        const TileRows mine = tile_rows(pos, row < places ? pair_of_pos[pos] : -1, gather_div, scatter);
        if (tid % 8 == 0) crow[row] = mine.c;
        ap[i] = mine.a >= 0 ? A + (size_t)mine.a * lda : nullptr;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int n = n0 + lr + 32 * i;
        wp[i] = n < N ? W + ((size_t)e * N + n) * K : nullptr;
    }
    const u32x4 zero = {0u, 0u, 0u, 0u};
    // MT 1: two steps' operands are on their way at any time (two sets of registers taking turns: one step's arithmetic
    // is shorter than a trip to the L2); MT 2 has registers for one set, and more arithmetic a step
    u32x4 va0[2 * MT], vw0[4], va1[2 * MT], vw1[4];
    auto fetch = [&](int k0, u32x4 (&va)[2 * MT], u32x4 (&vw)[4]) {
        const int k = k0 + lc;
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) va[i] = (ap[i] && k < K) ? *(const u32x4*)(ap[i] + k) : zero;
#pragma unroll
        for (int i = 0; i < 4; ++i) vw[i] = (wp[i] && k < K) ? *(const u32x4*)(wp[i] + k) : zero;
    };
    f32x4 acc[2 * MT][4];
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    int buf = 0;
    // one 64-deep step: the set's operands into LDS, the set asked for again `ahead` steps on, the step multiplied
    auto step = [&](int k0, u32x4 (&va)[2 * MT], u32x4 (&vw)[4], int ahead) {
#pragma unroll
        for (int i = 0; i < 2 * MT; ++i) *(u32x4*)(&As[buf][(lr + 32 * i) * EX_LD + lc]) = va[i];
#pragma unroll
        for (int i = 0; i < 4; ++i) *(u32x4*)(&Ws[buf][(lr + 32 * i) * EX_LD + lc]) = vw[i];
        __syncthreads();       // whoever writes this buffer again, two steps on, has passed the next step's barrier
        if (k0 + ahead * EX_BK < K) fetch(k0 + ahead * EX_BK, va, vw);
#pragma unroll
        for (int ks = 0; ks < EX_BK / 32; ++ks) {
            bf16x8 fa[2 * MT], fw[4];
#pragma unroll
            for (int i = 0; i < 2 * MT; ++i) fa[i] = *(const bf16x8*)(&As[buf][(wm * 32 * MT + i * 16 + r) * EX_LD + ks * 32 + g * 8]);
#pragma unroll
            for (int j = 0; j < 4; ++j) fw[j] = *(const bf16x8*)(&Ws[buf][(wn * 64 + j * 16 + r) * EX_LD + ks * 32 + g * 8]);
#pragma unroll
            for (int i = 0; i < 2 * MT; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
        }
        buf ^= 1;
    };
    fetch(0, va0, vw0);
    if (MT == 1) {
        if (EX_BK < K) fetch(EX_BK, va1, vw1);
        for (int k0 = 0; k0 < K; k0 += 2 * EX_BK) {
            step(k0, va0, vw0, 2);
            if (k0 + EX_BK < K) step(k0 + EX_BK, va1, vw1, 2);
        }
    } else {
        for (int k0 = 0; k0 < K; k0 += EX_BK) step(k0, va0, vw0, 1);
    }
    // a lane holds rows 4 g .. 4 g + 3 of column r in every 16 x 16 tile
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i)
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            const int m = crow[wm * 32 * MT + i * 16 + g * 4 + x];
            if (m < 0) continue;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int n = n0 + wn * 64 + j * 16 + r;
                if (n < N) store_f32(C + (size_t)m * ldc + n, expert_act<ACT>(acc[i][j][x]));
            }
        }
}

// ------------------------------------------------------------------ few rows: a pair streams its expert's matrix
// Steps of few rows (decoding) are bound by the bytes of the chosen experts' matrices.  grid (N / 16, pairs): a block of
// four waves makes 16 columns of one pair's row, a wave 4 of them: the operand row's share of a lane stays in registers
// (K up to 64 x 8 x EX_ROW_CHUNKS), the four matrix rows are read 16 bytes a lane, all loads of a column quartet in
// flight together.  C[pair] = act(A[pair / gather_div or pair] . W[chosen[pair]]^T).
#define EX_ROW_CHUNKS 16
template <typename TC, int ACT>
__global__ void __launch_bounds__(256)
expert_rows_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, const int* __restrict__ chosen,
                   int gather_div, TC* __restrict__ C, int ldc, int N, int K, int experts) {
    const int pair = blockIdx.y;
    const int e = chosen[pair];
    if (e < 0 || e >= experts) return;                       // (a choice without matrices: its row is left alone)
    const int wave = threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    const int n_first = (blockIdx.x * 4 + wave) * 4;
    if (n_first >= N) return;
    const bf16_t* ar = A + (size_t)(gather_div > 0 ? pair / gather_div : pair) * lda;
    const int chunks = (K + 511) / 512;                      // 16-byte chunks a lane holds of a row
    const u32x4 zero = {0u, 0u, 0u, 0u};
    u32x4 av[EX_ROW_CHUNKS];
#pragma unroll
    for (int c = 0; c < EX_ROW_CHUNKS; ++c) {
        const int k = (c * 64 + lane) * 8;
        av[c] = (c < chunks && k < K) ? *(const u32x4*)(ar + k) : zero;
    }
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    const bf16_t* wr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) wr[j] = W + ((size_t)e * N + min(n_first + j, N - 1)) * K;
#pragma unroll
    for (int c = 0; c < EX_ROW_CHUNKS; ++c) {
        if (c >= chunks) continue;                           // (uniform; the loop stays unrolled, the row in registers)
        const int k = (c * 64 + lane) * 8;
        u32x4 wv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) wv[j] = k < K ? __builtin_nontemporal_load((const u32x4*)(wr[j] + k)) : zero;
        const uint32_t aw[4] = {av[c].x, av[c].y, av[c].z, av[c].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t ww[4] = {wv[j].x, wv[j].y, wv[j].z, wv[j].w};
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                sum[j] = fmaf(__uint_as_float(aw[x] << 16), __uint_as_float(ww[x] << 16), sum[j]);
                sum[j] = fmaf(__uint_as_float(aw[x] & 0xffff0000u), __uint_as_float(ww[x] & 0xffff0000u), sum[j]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) sum[j] = wave_sum(sum[j]);
    if (lane < 4 && n_first + lane < N)
        store_f32(C + (size_t)pair * ldc + n_first + lane, expert_act<ACT>(lane == 0 ? sum[0] : lane == 1 ? sum[1] : lane == 2 ? sum[2] : sum[3]));
}

// Whether cisr_experts_rows takes a product: bf16 operands with 16-byte rows of at most 64 x 8 x EX_ROW_CHUNKS elements.
extern "C" int cisr_experts_rows_ok(int K, int lda, int pairs) {
    return K % 8 == 0 && lda % 8 == 0 && K <= 512 * EX_ROW_CHUNKS && pairs > 0 && pairs <= 65535;
}

extern "C" int cisr_experts_rows(const void* A, int lda, const void* W, const int* chosen, int gather_div, void* C, int ldc,
                                 int pairs, int N, int K, int act, int out_dtype, int experts, hipStream_t stream) {
    if (pairs <= 0 || N <= 0) return 0;
    if (!cisr_experts_rows_ok(K, lda, pairs) || ((uintptr_t)A) % 16 || ((uintptr_t)W) % 16) return (int)hipErrorInvalidValue;
    const dim3 grid((N + 15) / 16, pairs);
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    if (out_dtype == DT_F32) {
        if (act) expert_rows_kernel<float, 1><<<grid, 256, 0, stream>>>(a, lda, w, chosen, gather_div, (float*)C, ldc, N, K, experts);
        else expert_rows_kernel<float, 0><<<grid, 256, 0, stream>>>(a, lda, w, chosen, gather_div, (float*)C, ldc, N, K, experts);
    } else {
        if (act) expert_rows_kernel<bf16_t, 1><<<grid, 256, 0, stream>>>(a, lda, w, chosen, gather_div, (bf16_t*)C, ldc, N, K, experts);
        else expert_rows_kernel<bf16_t, 0><<<grid, 256, 0, stream>>>(a, lda, w, chosen, gather_div, (bf16_t*)C, ldc, N, K, experts);
    }
    return CISR_LAUNCH_CHECK();
}

// C[c row of place] = act(A[a row of place] . W[expert of the place's tile]^T); W is [experts, N, K].
// gather_div > 0: the operand's row of a place is pair / gather_div (a step's row), else the place itself;
// scatter: the result goes to row `pair`, else to the place.  dtype: of A and W; out_dtype: of C.
extern "C" int cisr_experts_gemm(const void* A, int lda, const void* W, const int* tile_expert, const int* pair_of_pos,
                                 int gather_div, int scatter, void* C, int ldc, int max_tiles, int N, int K, int act,
                                 int dtype, int out_dtype, hipStream_t stream) {
    if (max_tiles <= 0 || N <= 0) return 0;
    if (K <= 0 || max_tiles > 0x7fffff || (N + EX_TILE - 1) / EX_TILE > 65535 || (dtype == DT_F32 && out_dtype != DT_F32))
        return (int)hipErrorInvalidValue;
    const dim3 grid(max_tiles, (N + EX_TILE - 1) / EX_TILE);
    const long long wide_blocks = (long long)max_tiles * ((N + EX_BN - 1) / EX_BN);
    if (wide_blocks > 0x7ffffff0LL) return (int)hipErrorInvalidValue;
    const dim3 wide((unsigned)((wide_blocks + 7) / 8 * 8));
#define EX_ARGS tile_expert, pair_of_pos, gather_div, scatter
    if (dtype == DT_F32) {
        if (act) expert_gemm_fma_kernel<float, float, 1><<<grid, 256, 0, stream>>>((const float*)A, lda, (const float*)W, EX_ARGS, (float*)C, ldc, N, K);
        else expert_gemm_fma_kernel<float, float, 0><<<grid, 256, 0, stream>>>((const float*)A, lda, (const float*)W, EX_ARGS, (float*)C, ldc, N, K);
        return CISR_LAUNCH_CHECK();
    }
    const bool vec = K % 8 == 0 && lda % 8 == 0 && ((uintptr_t)A) % 16 == 0 && ((uintptr_t)W) % 16 == 0;
    const bf16_t* a = (const bf16_t*)A;
    const bf16_t* w = (const bf16_t*)W;
    if (vec) {
        // steps of many rows (an expert meets more than one tile as a rule): a block takes two tiles of one expert
#define EX_MFMA(TC, ACT) \
        do { if (max_tiles >= EX_PAIRED_FROM) expert_gemm_mfma_kernel<TC, ACT, 2><<<wide, 256, 0, stream>>>(a, lda, w, EX_ARGS, (TC*)C, ldc, N, K, max_tiles); \
             else expert_gemm_mfma_kernel<TC, ACT, 1><<<wide, 256, 0, stream>>>(a, lda, w, EX_ARGS, (TC*)C, ldc, N, K, max_tiles); } while (0)
        if (out_dtype == DT_F32) {
            if (act) EX_MFMA(float, 1);
            else EX_MFMA(float, 0);
        } else {
            if (act) EX_MFMA(bf16_t, 1);
            else EX_MFMA(bf16_t, 0);
        }
#undef EX_MFMA
    } else {
        if (out_dtype == DT_F32) {
            if (act) expert_gemm_fma_kernel<bf16_t, float, 1><<<grid, 256, 0, stream>>>(a, lda, w, EX_ARGS, (float*)C, ldc, N, K);
            else expert_gemm_fma_kernel<bf16_t, float, 0><<<grid, 256, 0, stream>>>(a, lda, w, EX_ARGS, (float*)C, ldc, N, K);
        } else {
            if (act) expert_gemm_fma_kernel<bf16_t, bf16_t, 1><<<grid, 256, 0, stream>>>(a, lda, w, EX_ARGS, (bf16_t*)C, ldc, N, K);
            else expert_gemm_fma_kernel<bf16_t, bf16_t, 0><<<grid, 256, 0, stream>>>(a, lda, w, EX_ARGS, (bf16_t*)C, ldc, N, K);
        }
    }
#undef EX_ARGS
    return CISR_LAUNCH_CHECK();
}
