// The minimal gated recurrent unit, element by element over a layer's channels:
//   z_t = sigmoid(a_t + bz), c_t = cand(b_t + bx), S_t = (1 - z_t) S_(t-1) + z_t c_t, out_t = S_t silu(g_t)
//   cand(u) = u + 1/2 for u >= 0, sigmoid(u) below
// with a_t, b_t, g_t three runs of `width` columns of a projection with float results.  The state is float and lives
// in the request's state slot; rows come as they are (portions and single tokens of several requests: seg_start,
// state_slots); a segment without rows (padding of a captured step) touches nothing.
//
// Single rows and short portions: a thread a (segment, channel) walks its rows in order, eight rows' operands asked
// for at a time.  Long portions are cut into pieces that waves of their own walk: a piece's rows compose to
// S_end = P S_start + Q (P the product of its 1 - z, Q its end state from zero); the states at the pieces' starts
// follow in order, then every piece is walked again from its true start state.  No division anywhere.
#include "common.h"

__device__ __forceinline__ float sigmoidf_(float v) { return 1.0f / (1.0f + expf(-v)); }

__device__ __forceinline__ void mingru_gates(float a, float b, float bz, float bx, float& z, float& c) {
    z = sigmoidf_(a + bz);
    const float u = b + bx;
    c = u >= 0.f ? u + 0.5f : sigmoidf_(u);
}

#define MG_AHEAD 8

// grid (channels / 64, segments): whole segments.
template <typename T>
__global__ void __launch_bounds__(64)
mingru_scan_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz, const float* __restrict__ bx,
                   float* __restrict__ state, int state_ld, const int* __restrict__ seg_start,
                   const int* __restrict__ state_slots, T* __restrict__ out, int width) {
    const int seg = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
    const int first = seg_start[seg], end = seg_start[seg + 1];
    if (end <= first || c >= width) return;
    float* sp = state + (size_t)state_slots[seg] * state_ld + c;
    float S = *sp;
    const float vbz = bz[c], vbx = bx[c];
    for (int t0 = first; t0 < end; t0 += MG_AHEAD) {
        float a[MG_AHEAD], b[MG_AHEAD], g[MG_AHEAD];
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            const float* pr = proj + (size_t)min(t0 + i, end - 1) * ld + c;
            a[i] = pr[0]; b[i] = pr[width]; g[i] = pr[2 * width];
        }
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            if (t0 + i >= end) break;
            float z, cand;
            mingru_gates(a[i], b[i], vbz, vbx, z, cand);
            S = (1.0f - z) * S + z * cand;
            store_f32(out + (size_t)(t0 + i) * width + c, S * (g[i] * sigmoidf_(g[i])));
        }
    }
    *sp = S;
}

// Pieces: every segment is cut into ceil(rows / piece) pieces of at most `piece` rows; the pieces of a step are numbered
// in the order of its segments.  Every block finds the rows of its piece from seg_start itself (steps with long
// portions have few segments).  Pass 1: grid (channels / 64, pieces): carry[piece] = (P, Q).
__device__ __forceinline__ bool piece_rows(const int* seg_start, int segments, int piece, int piece_index, int& seg, int& first, int& end) {
    // the piece_index-th piece of the step: segments in order, each cut into ceil(rows / piece) pieces
    int at = 0;
    for (int s = 0; s < segments; ++s) {
        const int f = seg_start[s], e = seg_start[s + 1];
        const int n = (e - f + piece - 1) / piece;
        if (piece_index < at + n) {
            seg = s;
            first = f + (piece_index - at) * piece;
            end = min(e, first + piece);
            return true;
        }
        at += n;
    }
    return false;
}

__global__ void __launch_bounds__(64)
mingru_pieces_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz, const float* __restrict__ bx,
                     const int* __restrict__ seg_start, int segments, int piece, float* __restrict__ carry, int width) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    int seg, first, end;
    if (!piece_rows(seg_start, segments, piece, blockIdx.y, seg, first, end) || c >= width) return;
    const float vbz = bz[c], vbx = bx[c];
    float P = 1.0f, Q = 0.f;
    for (int t0 = first; t0 < end; t0 += MG_AHEAD) {
        float a[MG_AHEAD], b[MG_AHEAD];
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            const float* pr = proj + (size_t)min(t0 + i, end - 1) * ld + c;
            a[i] = pr[0]; b[i] = pr[width];
        }
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            if (t0 + i >= end) break;
            float z, cand;
            mingru_gates(a[i], b[i], vbz, vbx, z, cand);
            P *= 1.0f - z;
            Q = (1.0f - z) * Q + z * cand;
        }
    }
    carry[((size_t)blockIdx.y * 2) * width + c] = P;
    carry[((size_t)blockIdx.y * 2 + 1) * width + c] = Q;
}

// Pass 2: grid (channels / 64, segments): the state at every piece's start (written over P), and the segment's end state.
__global__ void __launch_bounds__(64)
mingru_starts_kernel(const int* __restrict__ seg_start, int piece, float* __restrict__ carry, float* __restrict__ state,
                     int state_ld, const int* __restrict__ state_slots, int width) {
    const int seg = blockIdx.y, c = blockIdx.x * 64 + threadIdx.x;
    const int first = seg_start[seg], end = seg_start[seg + 1];
    if (end <= first || c >= width) return;
    int at = 0;
    for (int s = 0; s < seg; ++s) at += (seg_start[s + 1] - seg_start[s] + piece - 1) / piece;
    const int n = (end - first + piece - 1) / piece;
    float* sp = state + (size_t)state_slots[seg] * state_ld + c;
    float S = *sp;
    for (int p = 0; p < n; ++p) {
        const size_t i = ((size_t)(at + p) * 2) * width + c;
        const float P = carry[i], Q = carry[i + width];
        carry[i] = S;
        S = P * S + Q;
    }
    *sp = S;
}

// Pass 3: grid (channels / 64, pieces): the rows' results from the true start states.
template <typename T>
__global__ void __launch_bounds__(64)
mingru_results_kernel(const float* __restrict__ proj, int ld, const float* __restrict__ bz, const float* __restrict__ bx,
                      const int* __restrict__ seg_start, int segments, int piece, const float* __restrict__ carry,
                      T* __restrict__ out, int width) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    int seg, first, end;
    if (!piece_rows(seg_start, segments, piece, blockIdx.y, seg, first, end) || c >= width) return;
    const float vbz = bz[c], vbx = bx[c];
    float S = carry[((size_t)blockIdx.y * 2) * width + c];
    for (int t0 = first; t0 < end; t0 += MG_AHEAD) {
        float a[MG_AHEAD], b[MG_AHEAD], g[MG_AHEAD];
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            const float* pr = proj + (size_t)min(t0 + i, end - 1) * ld + c;
            a[i] = pr[0]; b[i] = pr[width]; g[i] = pr[2 * width];
        }
#pragma unroll
        for (int i = 0; i < MG_AHEAD; ++i) {
            if (t0 + i >= end) break;
            float z, cand;
            mingru_gates(a[i], b[i], vbz, vbx, z, cand);
            S = (1.0f - z) * S + z * cand;
            store_f32(out + (size_t)(t0 + i) * width + c, S * (g[i] * sigmoidf_(g[i])));
        }
    }
}

// proj float [rows, ld] = [a | b | g | ...] of `width` columns each; out [rows, width] float or bf16; state float
// [slots, state_ld].  piece 0: whole segments; else segments are walked in pieces of `piece` rows, carry float
// [2 * max_pieces * width] with max_pieces >= rows / piece + segments.
extern "C" int cisr_mingru_scan(const float* proj, int ld, const float* bz, const float* bx, float* state, int state_ld,
                                const int* seg_start, const int* state_slots, void* out, int rows, int segments, int width,
                                int piece, float* carry, int max_pieces, int out_dtype, hipStream_t stream) {
    if (rows <= 0 || segments <= 0) return 0;
    if (width <= 0 || ld < 3 * width || state_ld < width || segments > 65535) return (int)hipErrorInvalidValue;
    const int cblocks = (width + 63) / 64;
    if (piece <= 0) {
        const dim3 grid(cblocks, segments);
        if (out_dtype == DT_F32) mingru_scan_kernel<float><<<grid, 64, 0, stream>>>(proj, ld, bz, bx, state, state_ld, seg_start, state_slots, (float*)out, width);
        else mingru_scan_kernel<bf16_t><<<grid, 64, 0, stream>>>(proj, ld, bz, bx, state, state_ld, seg_start, state_slots, (bf16_t*)out, width);
        return CISR_LAUNCH_CHECK();
    }
    if (!carry || max_pieces < rows / piece + segments || max_pieces > 65535) return (int)hipErrorInvalidValue;
    mingru_pieces_kernel<<<dim3(cblocks, max_pieces), 64, 0, stream>>>(proj, ld, bz, bx, seg_start, segments, piece, carry, width);
    mingru_starts_kernel<<<dim3(cblocks, segments), 64, 0, stream>>>(seg_start, piece, carry, state, state_ld, state_slots, width);
    if (out_dtype == DT_F32) mingru_results_kernel<float><<<dim3(cblocks, max_pieces), 64, 0, stream>>>(proj, ld, bz, bx, seg_start, segments, piece, carry, (float*)out, width);
    else mingru_results_kernel<bf16_t><<<dim3(cblocks, max_pieces), 64, 0, stream>>>(proj, ld, bz, bx, seg_start, segments, piece, carry, (bf16_t*)out, width);
    return CISR_LAUNCH_CHECK();
}
