// The matrix memory with exponential gates (xLSTM's mLSTM), the parts around the linear scan.  Per head, with a log
// input gate i_t, a log forget gate f_t and a running maximum m (0 at a sequence's start):
//
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T          n_t likewise with k_t alone
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
//
// S and n are one state of C = vdim + 1 columns (n is the column of a value that is always 1), so the recurrence is the
// linear scan of recurrence_scan.inc with a decay a head and a step size: this file makes its operands and finishes
// its results.
//
//   gates      i_t = cap tanh((zi + bi) / cap), f_t = logsigmoid(cap tanh((zf + bf) / cap)) from the projections' float
//              results; the walk of m along a segment's rows (a thread a head; the maximum is the only chain); decay,
//              step and m_t a row and head; the values with their column of ones; m kept in the state slot
//   finish     o / denominator, each head divided by its root mean square, times a weight an element, times
//              sigmoid(gate), into the activations' type
// Everything here is float arithmetic.
#include "common.h"

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One block a segment.  zi / zf: [T, heads] views (row strides ldi / ldf); v [T, heads * V] (ldv); decay, step, top
// [T, heads]; vx [T, heads * (V + 1)]; m of a request at state + slot * slot_stride + head.
__global__ void __launch_bounds__(256)
mlstm_gates_kernel(const float* __restrict__ zi, int ldi, const float* __restrict__ zf, int ldf, const float* __restrict__ bi,
                   const float* __restrict__ bf, const float* __restrict__ v, int ldv, float* __restrict__ decay,
                   float* __restrict__ step, float* __restrict__ top, float* __restrict__ vx, float* __restrict__ state,
                   long long slot_stride, const int* __restrict__ seg_start, const int* __restrict__ state_slots, int heads, int V,
                   float cap) {
    const int seg = blockIdx.x;
    const int s0 = seg_start[seg], s1 = seg_start[seg + 1];
    if (s1 <= s0) return;                                            // (padding of a captured step)
    const int n = s1 - s0, C = V + 1;
    for (int i = threadIdx.x; i < n * heads; i += 256) {
        const int t = s0 + i / heads, h = i % heads;
        step[(size_t)t * heads + h] = cap * tanhf((zi[(size_t)t * ldi + h] + bi[h]) / cap);
        decay[(size_t)t * heads + h] = log_sigmoid(cap * tanhf((zf[(size_t)t * ldf + h] + bf[h]) / cap));
    }
    for (size_t i = threadIdx.x; i < (size_t)n * heads * C; i += 256) {
        const size_t t = s0 + i / ((size_t)heads * C);
        const int hc = (int)(i % ((size_t)heads * C)), h = hc / C, c = hc % C;
        vx[t * heads * C + hc] = c < V ? v[t * ldv + h * V + c] : 1.0f;
    }
    __syncthreads();
    float* ms = state + (long long)state_slots[seg] * slot_stride;
    for (int h = threadIdx.x; h < heads; h += 256) {
        float m = ms[h];
        for (int t = s0; t < s1; ++t) {
            const float f = decay[(size_t)t * heads + h], i = step[(size_t)t * heads + h];
            const float m_new = fmaxf(f + m, i);
            decay[(size_t)t * heads + h] = expf(f + m - m_new);
            step[(size_t)t * heads + h] = expf(i - m_new);
            top[(size_t)t * heads + h] = m_new;
            m = m_new;
        }
        ms[h] = m;
    }
}

extern "C" int cisr_mlstm_gates(const float* zi, int ldi, const float* zf, int ldf, const float* bi, const float* bf, const float* v,
                                int ldv, float* decay, float* step, float* top, float* vx, float* state, long long slot_stride,
                                const int* seg_start, const int* state_slots, int segments, int heads, int V, float cap,
                                hipStream_t stream) {
    if (segments <= 0) return 0;
    if (heads <= 0 || V <= 0 || !(cap > 0.f)) return (int)hipErrorInvalidValue;
    mlstm_gates_kernel<<<segments, 256, 0, stream>>>(zi, ldi, zf, ldf, bi, bf, v, ldv, decay, step, top, vx, state, slot_stride,
                                                     seg_start, state_slots, heads, V, cap);
    return CISR_LAUNCH_CHECK();
}

// A wave a (row, head): o [T, heads * (V + 1)] is the scan's result, its last column n . q.
template <typename T>
__global__ void __launch_bounds__(256)
mlstm_finish_kernel(const float* __restrict__ o, const float* __restrict__ top, const float* __restrict__ gate, int ldg,
                    const float* __restrict__ weight, T* __restrict__ out, int rows, int heads, int V, float eps, float floor_add) {
    const int item = blockIdx.x * 4 + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (item >= rows * heads) return;
    const int row = item / heads, h = item % heads, C = V + 1;
    const float* orow = o + ((size_t)row * heads + h) * C;
    const float den = fmaxf(fabsf(orow[V]), expf(-top[(size_t)row * heads + h])) + floor_add;
    float ss = 0.f;
    for (int c = lane; c < V; c += WAVE) { const float u = orow[c] / den; ss += u * u; }
    const float r = 1.0f / sqrtf(wave_sum(ss) / (float)V + eps);
    for (int c = lane; c < V; c += WAVE) {
        const int col = h * V + c;
        const float g = gate[(size_t)row * ldg + col];
        store_f32(out + (size_t)row * heads * V + col, orow[c] / den * r * weight[col] / (1.0f + expf(-g)));
    }
}

extern "C" int cisr_mlstm_finish(const float* o, const float* top, const float* gate, int ldg, const float* weight, void* out,
                                 int rows, int heads, int V, float eps, float floor_add, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (heads <= 0 || V <= 0 || ldg < heads * V) return (int)hipErrorInvalidValue;
    const unsigned blocks = (unsigned)(((long long)rows * heads + 3) / 4);
    if (dtype == DT_F32) mlstm_finish_kernel<float><<<blocks, 256, 0, stream>>>(o, top, gate, ldg, weight, (float*)out, rows, heads, V, eps, floor_add);
    else mlstm_finish_kernel<bf16_t><<<blocks, 256, 0, stream>>>(o, top, gate, ldg, weight, (bf16_t*)out, rows, heads, V, eps, floor_add);
    return CISR_LAUNCH_CHECK();
}
