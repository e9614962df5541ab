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
//              results and the values with their column of ones (a block a row); then the walk of m along a segment's
//              rows (a wave a segment and head, the rows dealt to its lanes in runs): decay, step and m_t a row and
//              head; m kept in the state slot
//   finish     o / denominator, each head divided by its root mean square, times a weight an element, times
//              sigmoid(gate), into the activations' type
// Everything here is float arithmetic.
#include "common.h"

__device__ __forceinline__ float log_sigmoid(float z) { return fminf(z, 0.f) - log1pf(expf(-fabsf(z))); }

// One block a row: the log gates of the row's heads (i into `step`, f into `decay`, for the walk below to turn into
// factors) and the row's values with their column of ones.  zi / zf: [T, heads] views (row strides ldi / ldf);
// v [T, heads * V] (ldv); vx [T, heads * (V + 1)].
// SINGLE: every segment has one row (row t is segment t), and the thread that makes a head's gates moves the head's
// running maximum on as well: no walk behind this kernel.
template <bool SINGLE>
__global__ void __launch_bounds__(256)
mlstm_rows_kernel(const float* __restrict__ zi, int ldi, const float* __restrict__ zf, int ldf, const float* __restrict__ bi,
                  const float* __restrict__ bf, const float* __restrict__ v, int ldv, float* __restrict__ decay,
                  float* __restrict__ step, float* __restrict__ vx, int heads, int V, float cap, float* __restrict__ top,
                  float* __restrict__ state, long long slot_stride, const int* __restrict__ seg_start,
                  const int* __restrict__ state_slots, int segments) {
    const size_t t = blockIdx.x;
    const int C = V + 1;
    const bool live = SINGLE && (int)t < segments && seg_start[t + 1] > seg_start[t];        // (else: padding of a captured step)
    for (int h = threadIdx.x; h < heads; h += 256) {
        const float i = cap * tanhf((zi[t * ldi + h] + bi[h]) / cap);
        const float f = log_sigmoid(cap * tanhf((zf[t * ldf + h] + bf[h]) / cap));
        if (!SINGLE) { step[t * heads + h] = i; decay[t * heads + h] = f; continue; }
        if (!live) continue;
        float* ms = state + (long long)state_slots[t] * slot_stride + h;
        const float m = *ms, m_new = fmaxf(f + m, i);
        decay[t * heads + h] = expf(f + m - m_new);
        step[t * heads + h] = expf(i - m_new);
        top[t * heads + h] = m_new;
        *ms = m_new;
    }
    for (int hc = threadIdx.x; hc < heads * C; hc += 256) {
        const int h = hc / C, c = hc % C;
        vx[t * heads * C + hc] = c < V ? v[t * ldv + h * V + c] : 1.0f;
    }
}

// The walk of the running maximum, a wave a (segment, head): m' = max(f + m, i) along the segment's rows is the map
// x -> max(a + x, b) with (a, b) = (f, i), and two such maps compose to one: later o earlier = (a1 + a2, max(a2 + b1,
// b2)).  A lane composes its run of consecutive rows, the lanes' maps meet in a scan over the wave, and every lane walks
// its run again from the maximum it starts with, turning the log gates into the factors of the state's update
// (decay = exp(f + m - m'), step = exp(i - m')) and leaving m' (`top`).  m of a request at state + slot * slot_stride + head.
__global__ void __launch_bounds__(64)
mlstm_walk_kernel(float* __restrict__ decay, float* __restrict__ step, float* __restrict__ top, float* __restrict__ state,
                  long long slot_stride, const int* __restrict__ seg_start, const int* __restrict__ state_slots, int heads) {
    const int seg = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int s0 = seg_start[seg], s1 = seg_start[seg + 1];
    if (s1 <= s0) return;                                            // (padding of a captured step)
    float* ms = state + (long long)state_slots[seg] * slot_stride + h;
    const int n = s1 - s0, per = (n + WAVE - 1) / WAVE;
    const int t0 = min(s0 + lane * per, s1), t1 = min(t0 + per, s1);
    float A = 0.f, B = -INFINITY;                                    // the identity map
    for (int t = t0; t < t1; ++t) {
        const float f = decay[(size_t)t * heads + h], i = step[(size_t)t * heads + h];
        B = fmaxf(f + B, i);
        A += f;
    }
#pragma unroll
    for (int off = 1; off < WAVE; off <<= 1) {
        const float Ap = __shfl_up(A, off, WAVE), Bp = __shfl_up(B, off, WAVE);
        if (lane >= off) { B = fmaxf(A + Bp, B); A += Ap; }
    }
    const float m0 = *ms;
    const float Ab = __shfl_up(A, 1, WAVE), Bb = __shfl_up(B, 1, WAVE);
    float m = lane == 0 ? m0 : fmaxf(Ab + m0, Bb);                   // the maximum before this lane's first row
    for (int t = t0; t < t1; ++t) {
        const float f = decay[(size_t)t * heads + h], i = step[(size_t)t * heads + h];
        const float m_new = fmaxf(f + m, i);
        decay[(size_t)t * heads + h] = expf(f + m - m_new);
        step[(size_t)t * heads + h] = expf(i - m_new);
        top[(size_t)t * heads + h] = m_new;
        m = m_new;
    }
    if (t1 == s1 && t0 < t1) *ms = m;                                // (the lane of the segment's last row)
}

extern "C" int cisr_mlstm_gates(const float* zi, int ldi, const float* zf, int ldf, const float* bi, const float* bf, const float* v,
                                int ldv, float* decay, float* step, float* top, float* vx, float* state, long long slot_stride,
                                const int* seg_start, const int* state_slots, int rows, int segments, int heads, int V, float cap,
                                int single_rows, hipStream_t stream) {
    if (segments <= 0 || rows <= 0) return 0;
    if (heads <= 0 || heads > 65535 || V <= 0 || !(cap > 0.f)) return (int)hipErrorInvalidValue;
    if (single_rows) {
        mlstm_rows_kernel<true><<<rows, 256, 0, stream>>>(zi, ldi, zf, ldf, bi, bf, v, ldv, decay, step, vx, heads, V, cap, top, state,
                                                          slot_stride, seg_start, state_slots, segments);
        return CISR_LAUNCH_CHECK();
    }
    mlstm_rows_kernel<false><<<rows, 256, 0, stream>>>(zi, ldi, zf, ldf, bi, bf, v, ldv, decay, step, vx, heads, V, cap, top, state,
                                                       slot_stride, seg_start, state_slots, segments);
    int err = CISR_LAUNCH_CHECK();
    if (err) return err;
    mlstm_walk_kernel<<<dim3(segments, heads), 64, 0, stream>>>(decay, step, top, state, slot_stride, seg_start, state_slots, heads);
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
