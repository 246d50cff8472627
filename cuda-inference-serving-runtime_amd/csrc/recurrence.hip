// Kernels of mixers that carry a fixed-size state per request instead of keys and values:
//
//   linear scan     S_t = diag(a_t) S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t   per head, S [R, C] float in the state slot
//                   of the row's request; a_t a vector over the R rows (a decay per key channel) or one number a head
//                   (state-space duality), q and k of a group of heads shared or not, v optionally times a step size
//   short conv      a causal convolution per channel over the last `taps` inputs, the taps - 1 inputs before a portion
//                   taken from the state slot, + bias, silu; with it the step sizes softplus(dt + bias) and the decays
//                   exp(-exp(A_log) dt) of a state-space layer
//   decay gates     a = sigmoid(z + bias)^(1 / tau) as exp(log sigmoid / tau)
//   group norm gate the output of such a mixer: RMS norm over equal parts of a row, times a weight, with a silu gate
//                   before or after the norm and an optional skip term D x
//
// Every kernel takes a step's rows as they come: portions of several requests side by side, single tokens among
// them.  seg_start[s] .. seg_start[s + 1] are the rows of segment s, state_slots[s] its request's slot; a segment
// without rows (padding of a captured step) touches nothing.  All of it is float arithmetic on float data: what
// enters a recurrence is 32-bit in every mode.
#include "common.h"
#include "recurrence_scan.inc"

// ------------------------------------------------------------------------------------------------ linear scan
// (the kernel: recurrence_scan.inc; one source file a tile width)
// Floats of `carry` and of `carry_decay` that a launch over `rows` rows in pieces of `piece` rows needs.
extern "C" long long cisr_linear_scan_carry(int rows, int piece, int heads, int R, int C, int vec, long long* decay_floats) {
    const long long pieces = piece > 0 ? (rows + piece - 1) / piece : 0;     // (the segments' pieces but their last are at most rows / piece)
    if (decay_floats) *decay_floats = pieces * heads * (vec ? R : 1);
    return pieces * heads * R * C;
}

int cisr_scan_launch_c4(const ScanArgs& p, int segments, bool vec, hipStream_t stream);
int cisr_scan_launch_c8(const ScanArgs& p, int segments, bool vec, hipStream_t stream);
int cisr_scan_launch_c16(const ScanArgs& p, int segments, bool vec, hipStream_t stream);

// cols: 4, 8 or 16 columns a wave (the caller's rule: fewer columns are more waves for the same head).  piece > 0:
// segments longer than `piece` rows are walked in pieces of that many rows side by side (three launches; `rows` is the
// number of rows of the step, carry / carry_decay as cisr_linear_scan_carry says); piece 0: a wave walks a whole segment.
extern "C" int cisr_linear_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                const float* a, int lda, int vec, const float* vs, int ldvs, float* out, int ldo,
                                float* state, long long slot_stride, const int* seg_start, const int* state_slots,
                                int segments, int heads, int R, int C, int share, float q_scale, int cols,
                                int rows, int piece, float* carry, float* carry_decay, hipStream_t stream) {
    if (segments <= 0 || heads <= 0) return 0;
    if (R <= 0 || C <= 0 || share <= 0 || heads % share || heads > 65535 || (cols != 4 && cols != 8 && cols != 16) ||
        piece < 0 || (piece > 0 && (!carry || !carry_decay || rows <= 0)))
        return (int)hipErrorInvalidValue;
    ScanArgs p{q, ldq, k, ldk, v, ldv, a, lda, vs, ldvs, out, ldo, state, slot_stride, seg_start, state_slots, R, C, share, heads,
               q_scale, piece, piece > 0 ? (rows + piece - 1) / piece : 1, 0, carry, carry_decay};
    if ((C + cols - 1) / cols > 65535 || R > 256 || (piece > 0 && segments > 65535)) return (int)hipErrorInvalidValue;
    if (cols == 4) return cisr_scan_launch_c4(p, segments, vec, stream);
    if (cols == 8) return cisr_scan_launch_c8(p, segments, vec, stream);
    return cisr_scan_launch_c16(p, segments, vec, stream);
}

// ------------------------------------------------------------------------------------------------ short conv
#define MAX_TAPS 16

// in[t * ld + first + ch], ch < channels: the convolution's inputs of row t.  conv_state[slot * slot_stride +
// j * channels + ch], j < taps - 1: the inputs of the request's last taps - 1 tokens, oldest first.
// out[t * channels + ch] = silu(bias[ch] + sum_j w[ch * taps + j] * input(t - (taps - 1) + j)).
// Index channels + h, h < heads (if heads > 0): step[t * heads + h] = softplus(in[t * ld + dt_first + h] + dt_bias[h]),
// decay[t * heads + h] = exp(-exp(a_log[h]) * step).
// SINGLE: every segment has one row (a step of single tokens), so the thread of a (row, channel) is the only one that
// reads that channel of its request's state, and it moves the state on itself: no second launch.
template <bool SINGLE>
__global__ void __launch_bounds__(256)
conv_silu_kernel(const float* __restrict__ in, int ld, int first, const float* __restrict__ w, const float* __restrict__ bias,
                 float* conv_state, long long slot_stride, float* __restrict__ out,
                 const int* __restrict__ seg_of_row, const int* __restrict__ seg_start, const int* __restrict__ state_slots,
                 int channels, int taps, int heads, int dt_first, const float* __restrict__ dt_bias,
                 const float* __restrict__ a_log, float* __restrict__ step, float* __restrict__ decay) {
    const int t = blockIdx.x;
    const int idx = blockIdx.y * 256 + threadIdx.x;
    const int seg = seg_of_row[t];
    if (seg < 0 || idx >= channels + heads) return;
    if (idx >= channels) {
        const int h = idx - channels;
        const float z = in[(size_t)t * ld + dt_first + h] + dt_bias[h];
        const float dt = z > 20.f ? z : log1pf(expf(z));
        step[(size_t)t * heads + h] = dt;
        decay[(size_t)t * heads + h] = expf(-expf(a_log[h]) * dt);
        return;
    }
    const int rel = t - seg_start[seg];
    float* st = conv_state + (long long)state_slots[seg] * slot_stride;
    float y = bias ? bias[idx] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = rel - (taps - 1) + j;
        const float x = src >= 0 ? in[(size_t)(t - rel + src) * ld + first + idx] : st[(size_t)(taps - 1 + src) * channels + idx];
        y += w[(size_t)idx * taps + j] * x;
        if (SINGLE && j > 0) st[(size_t)(j - 1) * channels + idx] = x;     // (input j of this row is input j - 1 of the next)
    }
    out[(size_t)t * channels + idx] = y / (1.0f + expf(-y));
}

// After the convolution has read it: the state becomes the last taps - 1 inputs of (state, portion).
__global__ void __launch_bounds__(256)
conv_state_kernel(const float* __restrict__ in, int ld, int first, float* __restrict__ conv_state, long long slot_stride,
                  const int* __restrict__ seg_start, const int* __restrict__ state_slots, int channels, int taps) {
    const int seg = blockIdx.x, ch = blockIdx.y * 256 + threadIdx.x;
    const int t0 = seg_start[seg], count = seg_start[seg + 1] - t0;
    if (count <= 0 || ch >= channels) return;
    float* st = conv_state + (long long)state_slots[seg] * slot_stride;
    float keep[MAX_TAPS];
#pragma unroll
    for (int i = 0; i < MAX_TAPS; ++i) {
        if (i >= taps - 1) break;
        const int src = count - (taps - 1) + i;
        keep[i] = src >= 0 ? in[(size_t)(t0 + src) * ld + first + ch] : st[(size_t)(taps - 1 + src) * channels + ch];
    }
#pragma unroll
    for (int i = 0; i < MAX_TAPS; ++i) {
        if (i >= taps - 1) break;
        st[(size_t)i * channels + ch] = keep[i];
    }
}

extern "C" int cisr_conv_silu(const float* in, int ld, int first, const float* w, const float* bias, float* conv_state,
                              long long slot_stride, float* out, const int* seg_of_row, const int* seg_start,
                              const int* state_slots, int rows, int segments, int channels, int taps, int heads,
                              int dt_first, const float* dt_bias, const float* a_log, float* step, float* decay,
                              int single_rows, hipStream_t stream) {
    if (rows <= 0 || segments <= 0) return 0;
    if (channels <= 0 || taps < 1 || taps > MAX_TAPS || heads < 0 || segments > 65535) return (int)hipErrorInvalidValue;
    const dim3 grid(rows, (channels + heads + 255) / 256);
    if (single_rows) {       // `single_rows`: the caller knows that no segment has more than one row
        conv_silu_kernel<true><<<grid, 256, 0, stream>>>(in, ld, first, w, bias, conv_state, slot_stride,
            out, seg_of_row, seg_start, state_slots, channels, taps, heads, dt_first, dt_bias, a_log, step, decay);
        return CISR_LAUNCH_CHECK();
    }
    conv_silu_kernel<false><<<grid, 256, 0, stream>>>(in, ld, first, w, bias, conv_state, slot_stride,
        out, seg_of_row, seg_start, state_slots, channels, taps, heads, dt_first, dt_bias, a_log, step, decay);
    int err = CISR_LAUNCH_CHECK();
    if (err || taps == 1) return err;
    conv_state_kernel<<<dim3(segments, (channels + 255) / 256), 256, 0, stream>>>(in, ld, first, conv_state, slot_stride, seg_start,
        state_slots, channels, taps);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------------------ decay gates
// a[i] = sigmoid(z[t * ld + c] + bias[c])^(1 / tau) = exp(log sigmoid(.) / tau), log sigmoid(u) = min(u, 0) - log1p(exp(-|u|))
__global__ void decay_gate_kernel(const float* __restrict__ z, int ld, const float* __restrict__ bias, float* __restrict__ a,
                                  int cols, size_t n, float inv_tau) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / cols;
    const int c = (int)(i % cols);
    const float u = z[t * ld + c] + (bias ? bias[c] : 0.f);
    a[i] = expf((fminf(u, 0.f) - log1pf(expf(-fabsf(u)))) * inv_tau);
}

// The same with z = up . low made on the way: z[t, c] = sum_r up_t[r * cols + c] * low[t * ld + r] (the second half of a
// low-rank projection, its matrix transposed so that neighbouring lanes read neighbouring words; the first half came
// out of the mixer's fused input product).
__global__ void decay_gate_low_rank_kernel(const float* __restrict__ low, int ld, int rank, const float* __restrict__ up,
                                           const float* __restrict__ bias, float* __restrict__ a, int cols, size_t n, float inv_tau) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const size_t t = i / cols;
    const int c = (int)(i % cols);
    const float* lo = low + t * ld;
    const float* w = up + c;
    float u = bias ? bias[c] : 0.f;
#pragma unroll 4
    for (int r = 0; r < rank; ++r) u += w[(size_t)r * cols] * lo[r];
    a[i] = expf((fminf(u, 0.f) - log1pf(expf(-fabsf(u)))) * inv_tau);
}

extern "C" int cisr_decay_gate_low_rank(const float* low, int ld, int rank, const float* up, const float* bias, float* a,
                                        int rows, int cols, float tau, hipStream_t stream) {
    const size_t n = (size_t)rows * cols;
    if (n == 0) return 0;
    if (!(tau > 0.f) || rank <= 0) return (int)hipErrorInvalidValue;
    decay_gate_low_rank_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(low, ld, rank, up, bias, a, cols, n, 1.0f / tau);
    return CISR_LAUNCH_CHECK();
}

extern "C" int cisr_decay_gate(const float* z, int ld, const float* bias, float* a, int rows, int cols, float tau,
                               hipStream_t stream) {
    const size_t n = (size_t)rows * cols;
    if (n == 0) return 0;
    if (!(tau > 0.f)) return (int)hipErrorInvalidValue;
    decay_gate_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(z, ld, bias, a, cols, n, 1.0f / tau);
    return CISR_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------------------ group norm gate
// Row t of y [T, groups * size] in `groups` equal parts; part g, element d, i = g * size + d:
//   u = y[t, i] + (skip ? skip[i / skip_span] * x[t * ldx + i] : 0)
//   GATE_FIRST:  u *= silu(gate[t * ldg + i]);  out = u / rms(part) * w[shared ? d : i]
//   else:        out = u / rms(part) * w[shared ? d : i] * silu(gate[t * ldg + i])
// A block of NT threads a (row, part): a wave for parts of up to 256 elements, four waves up to 2,048, sixteen beyond.
// KEEP: the part's elements (after the skip term and the gate before the norm) wait in LDS for their scale, so every
// input is read once; else (parts of more than 12,288 elements) they are made a second time.
template <typename T, bool GATE_FIRST, int NT, bool KEEP>
__global__ void __launch_bounds__(NT)
group_norm_gate_kernel(const float* __restrict__ y, const float* __restrict__ gate, int ldg, const float* __restrict__ w,
                       int shared, const float* __restrict__ skip, int skip_span, const float* __restrict__ x, int ldx,
                       T* __restrict__ out, int size, float eps) {
    __shared__ float red[NT / WAVE];
    extern __shared__ float kept[];
    const int t = blockIdx.x, g = blockIdx.y, groups = gridDim.y, lane = threadIdx.x;
    const size_t base = (size_t)t * groups * size + (size_t)g * size;
    const int col0 = g * size;
    auto element = [&](int d) {
        float u = y[base + d];
        if (skip) u += skip[(col0 + d) / skip_span] * x[(size_t)t * ldx + col0 + d];
        if (GATE_FIRST) { const float z = gate[(size_t)t * ldg + col0 + d]; u *= z / (1.0f + expf(-z)); }
        return u;
    };
    float ss = 0.f;
    for (int d = lane; d < size; d += NT) {
        const float u = element(d);
        if (KEEP) kept[d] = u;
        ss += u * u;
    }
    const float scale = 1.0f / sqrtf((NT == WAVE ? wave_sum(ss) : block_sum<NT>(ss, red)) / (float)size + eps);
    for (int d = lane; d < size; d += NT) {
        float u = (KEEP ? kept[d] : element(d)) * scale * w[shared ? d : col0 + d];     // (a thread reads back what it wrote)
        if (!GATE_FIRST) { const float z = gate[(size_t)t * ldg + col0 + d]; u *= z / (1.0f + expf(-z)); }
        store_f32(out + base + d, u);
    }
}

template <typename T, bool GATE_FIRST>
static void launch_group_norm_gate(const float* y, const float* gate, int ldg, const float* w, int shared, const float* skip,
                                   int skip_span, const float* x, int ldx, T* out, int rows, int groups, int size, float eps,
                                   hipStream_t stream) {
    const dim3 grid(rows, groups);
    const size_t lds = (size_t)size * sizeof(float);
#define GNG(NT, KEEP) group_norm_gate_kernel<T, GATE_FIRST, NT, KEEP><<<grid, NT, KEEP ? lds : 0, stream>>>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, out, size, eps)
    if (size <= 256) GNG(64, true);
    else if (size <= 2048) GNG(256, true);
    else if (size <= 12288) GNG(1024, true);
    else GNG(1024, false);
#undef GNG
}

extern "C" int cisr_group_norm_gate(const float* y, const float* gate, int ldg, const float* w, int shared, const float* skip,
                                    int skip_span, const float* x, int ldx, void* out, int rows, int groups, int size,
                                    float eps, int gate_first, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (groups <= 0 || groups > 65535 || size <= 0 || (skip && (skip_span <= 0 || !x))) return (int)hipErrorInvalidValue;
    if (dtype == DT_F32) {
        if (gate_first) launch_group_norm_gate<float, true>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, (float*)out, rows, groups, size, eps, stream);
        else launch_group_norm_gate<float, false>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, (float*)out, rows, groups, size, eps, stream);
    } else {
        if (gate_first) launch_group_norm_gate<bf16_t, true>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, (bf16_t*)out, rows, groups, size, eps, stream);
        else launch_group_norm_gate<bf16_t, false>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, (bf16_t*)out, rows, groups, size, eps, stream);
    }
    return CISR_LAUNCH_CHECK();
}
