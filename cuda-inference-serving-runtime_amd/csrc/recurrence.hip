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

// ------------------------------------------------------------------------------------------------ linear scan
struct ScanArgs {
    const float* q; int ldq;          // q[t * ldq + (head / share) * R + r]
    const float* k; int ldk;          // k[t * ldk + (head / share) * R + r]
    const float* v; int ldv;          // v[t * ldv + head * C + c]
    const float* a; int lda;          // VEC: a[t * lda + head * R + r]; else a[t * lda + head]
    const float* vs; int ldvs;        // null, or the step size vs[t * ldvs + head] that multiplies v
    float* out; int ldo;              // out[t * ldo + head * C + c]
    float* state; long long slot_stride;   // state + slot * slot_stride + (head * R + r) * C + c
    const int* seg_start; const int* state_slots;
    int R, C, share;
    float q_scale;
};

// A wave a (segment, head, tile of COLS columns).  Lane l owns column l % COLS and the rows l / COLS + (64 / COLS) i,
// i < RPT, of the state, in registers, and walks the segment's rows in order; the products of a column meet over the
// 64 / COLS lanes that share it.  Columns of S are independent, so a head is as many waves as it has tiles.
template <int COLS, int RPT, bool VEC>
__global__ void __launch_bounds__(64) linear_scan_kernel(ScanArgs p) {
    constexpr int NG = WAVE / COLS;
    const int seg = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int t0 = p.seg_start[seg], t1 = p.seg_start[seg + 1];
    if (t1 <= t0) return;
    const int c = blockIdx.z * COLS + lane % COLS, rg = lane / COLS;
    const bool col_ok = c < p.C;
    const int cc = col_ok ? c : p.C - 1;
    const int R = p.R, C = p.C;
    float* state = p.state + (long long)p.state_slots[seg] * p.slot_stride + (size_t)head * R * C;
    const float* qh = p.q + (size_t)(head / p.share) * R;
    const float* kh = p.k + (size_t)(head / p.share) * R;
    const float* ah = p.a + (VEC ? (size_t)head * R : (size_t)head);
    const float* vh = p.v + (size_t)head * C + cc;
    float S[RPT];
    int rows[RPT];
    bool ok[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const int r = rg + NG * i;
        ok[i] = r < R;
        rows[i] = ok[i] ? r : R - 1;
        S[i] = ok[i] ? state[(size_t)rows[i] * C + cc] : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        float v = vh[(size_t)t * p.ldv];
        if (p.vs) v *= p.vs[(size_t)t * p.ldvs + head];
        const float a1 = VEC ? 0.f : ah[(size_t)t * p.lda];
        const float* qt = qh + (size_t)t * p.ldq;
        const float* kt = kh + (size_t)t * p.ldk;
        const float* at = ah + (size_t)t * p.lda;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < RPT; ++i) {
            const float kk = ok[i] ? kt[rows[i]] : 0.f;      // (a row past R stays zero and adds nothing)
            const float aa = VEC ? at[rows[i]] : a1;
            S[i] = aa * S[i] + kk * v;
            acc += S[i] * qt[rows[i]];
        }
#pragma unroll
        for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off, WAVE);
        if (rg == 0 && col_ok) p.out[(size_t)t * p.ldo + (size_t)head * C + c] = acc * p.q_scale;
    }
    if (col_ok) {
#pragma unroll
        for (int i = 0; i < RPT; ++i)
            if (ok[i]) state[(size_t)rows[i] * C + c] = S[i];
    }
}

template <int COLS, int RPT>
static int launch_scan(const ScanArgs& p, int segments, int heads, bool vec, hipStream_t stream) {
    const dim3 grid(segments, heads, (p.C + COLS - 1) / COLS);
    if (vec) linear_scan_kernel<COLS, RPT, true><<<grid, 64, 0, stream>>>(p);
    else linear_scan_kernel<COLS, RPT, false><<<grid, 64, 0, stream>>>(p);
    return CISR_LAUNCH_CHECK();
}

// cols: 4, 8 or 16 columns a wave (the caller's rule: fewer columns are more waves for the same head).
extern "C" int cisr_linear_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                const float* a, int lda, int vec, const float* vs, int ldvs, float* out, int ldo,
                                float* state, long long slot_stride, const int* seg_start, const int* state_slots,
                                int segments, int heads, int R, int C, int share, float q_scale, int cols,
                                hipStream_t stream) {
    if (segments <= 0 || heads <= 0) return 0;
    if (R <= 0 || C <= 0 || share <= 0 || heads % share || heads > 65535 || (cols != 4 && cols != 8 && cols != 16))
        return (int)hipErrorInvalidValue;
    ScanArgs p{q, ldq, k, ldk, v, ldv, a, lda, vs, ldvs, out, ldo, state, slot_stride, seg_start, state_slots, R, C, share, q_scale};
    const int per = (R + (WAVE / cols) - 1) / (WAVE / cols);    // rows a lane
    if ((C + cols - 1) / cols > 65535) return (int)hipErrorInvalidValue;
#define SCAN_CASE(COLS) \
    if (cols == COLS) { \
        if (per <= 2) return launch_scan<COLS, 2>(p, segments, heads, vec, stream); \
        if (per <= 4) return launch_scan<COLS, 4>(p, segments, heads, vec, stream); \
        if (per <= 8) return launch_scan<COLS, 8>(p, segments, heads, vec, stream); \
        if (per <= 16) return launch_scan<COLS, 16>(p, segments, heads, vec, stream); \
        if (per <= 32) return launch_scan<COLS, 32>(p, segments, heads, vec, stream); \
        if (per <= 64) return launch_scan<COLS, 64>(p, segments, heads, vec, stream); \
        return (int)hipErrorInvalidValue; \
    }
    SCAN_CASE(4)
    SCAN_CASE(8)
    SCAN_CASE(16)
#undef SCAN_CASE
    return (int)hipErrorInvalidValue;
}

// ------------------------------------------------------------------------------------------------ short conv
#define MAX_TAPS 16

// in[t * ld + first + ch], ch < channels: the convolution's inputs of row t.  conv_state[slot * slot_stride +
// j * channels + ch], j < taps - 1: the inputs of the request's last taps - 1 tokens, oldest first.
// out[t * channels + ch] = silu(bias[ch] + sum_j w[ch * taps + j] * input(t - (taps - 1) + j)).
// Index channels + h, h < heads (if heads > 0): step[t * heads + h] = softplus(in[t * ld + dt_first + h] + dt_bias[h]),
// decay[t * heads + h] = exp(-exp(a_log[h]) * step).
__global__ void __launch_bounds__(256)
conv_silu_kernel(const float* __restrict__ in, int ld, int first, const float* __restrict__ w, const float* __restrict__ bias,
                 const float* __restrict__ conv_state, long long slot_stride, float* __restrict__ out,
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
    const float* st = conv_state + (long long)state_slots[seg] * slot_stride;
    float y = bias ? bias[idx] : 0.f;
    for (int j = 0; j < taps; ++j) {
        const int src = rel - (taps - 1) + j;
        const float x = src >= 0 ? in[(size_t)(t - rel + src) * ld + first + idx] : st[(size_t)(taps - 1 + src) * channels + idx];
        y += w[(size_t)idx * taps + j] * x;
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
                              hipStream_t stream) {
    if (rows <= 0 || segments <= 0) return 0;
    if (channels <= 0 || taps < 1 || taps > MAX_TAPS || heads < 0 || segments > 65535) return (int)hipErrorInvalidValue;
    conv_silu_kernel<<<dim3(rows, (channels + heads + 255) / 256), 256, 0, stream>>>(in, ld, first, w, bias, conv_state, slot_stride,
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
// A wave a (row, part); the part is read twice.
template <typename T, bool GATE_FIRST>
__global__ void __launch_bounds__(64)
group_norm_gate_kernel(const float* __restrict__ y, const float* __restrict__ gate, int ldg, const float* __restrict__ w,
                       int shared, const float* __restrict__ skip, int skip_span, const float* __restrict__ x, int ldx,
                       T* __restrict__ out, int size, float eps) {
    const int t = blockIdx.x, g = blockIdx.y, groups = gridDim.y, lane = threadIdx.x;
    const size_t base = (size_t)t * groups * size + (size_t)g * size;
    const int col0 = g * size;
    float ss = 0.f;
    for (int d = lane; d < size; d += WAVE) {
        float u = y[base + d];
        if (skip) u += skip[(col0 + d) / skip_span] * x[(size_t)t * ldx + col0 + d];
        if (GATE_FIRST) { const float z = gate[(size_t)t * ldg + col0 + d]; u *= z / (1.0f + expf(-z)); }
        ss += u * u;
    }
    const float scale = 1.0f / sqrtf(wave_sum(ss) / (float)size + eps);
    for (int d = lane; d < size; d += WAVE) {
        float u = y[base + d];
        if (skip) u += skip[(col0 + d) / skip_span] * x[(size_t)t * ldx + col0 + d];
        const float z = gate[(size_t)t * ldg + col0 + d];
        const float s = z / (1.0f + expf(-z));
        if (GATE_FIRST) u *= s;
        u *= scale * w[shared ? d : col0 + d];
        if (!GATE_FIRST) u *= s;
        store_f32(out + base + d, u);
    }
}

extern "C" int cisr_group_norm_gate(const float* y, const float* gate, int ldg, const float* w, int shared, const float* skip,
                                    int skip_span, const float* x, int ldx, void* out, int rows, int groups, int size,
                                    float eps, int gate_first, int dtype, hipStream_t stream) {
    if (rows <= 0) return 0;
    if (groups <= 0 || groups > 65535 || size <= 0 || (skip && (skip_span <= 0 || !x))) return (int)hipErrorInvalidValue;
    const dim3 grid(rows, groups);
#define GNG(T, GF) group_norm_gate_kernel<T, GF><<<grid, 64, 0, stream>>>(y, gate, ldg, w, shared, skip, skip_span, x, ldx, (T*)out, size, eps)
    if (dtype == DT_F32) { if (gate_first) GNG(float, true); else GNG(float, false); }
    else { if (gate_first) GNG(bf16_t, true); else GNG(bf16_t, false); }
#undef GNG
    return CISR_LAUNCH_CHECK();
}
