// The gated delta rule, per head, over the rows of a step as they come (portions and single tokens of several
// requests), S [R, C] float in the state slot of the row's request:
//
//   S <- g_t S;  u = beta_t (v_t - S^T k_t);  S <- S + k_t u^T;  o_t = S^T q_t
//
// g_t one decay a head, beta_t = sigmoid(b_t) one write strength a head, q and k shared by `share` heads.  The
// columns of S go their own ways (column c needs k, q, v_t[c] and itself only), so a head is as many waves as it has
// tiles of columns.  Both products with the state are taken from the state as the row finds it,
//   S^T k = g (S_old^T k),   o = g (S_old^T q) + (k . q) u,
// so that a row costs one meeting of the lanes that share a column instead of two.  The lanes that share a column are
// neighbours, so their sums meet by moves inside a row of 16 lanes, without a trip through LDS.
// With it: the unit vectors x / sqrt(sum(x^2) + eps) * scale of the heads of a row (q and k of this rule).
#include "common.h"

struct DeltaArgs {
    const float* q; int ldq;          // q[t * ldq + (head / share) * R + r]
    const float* k; int ldk;
    const float* v; int ldv;          // v[t * ldv + head * C + c]
    const float* g; int ldg;          // g[t * ldg + head]
    const float* b; int ldb;          // b[t * ldb + head], beta = sigmoid(b)
    float* out; int ldo;
    float* state; long long slot_stride;
    const int* seg_start; const int* state_slots;
    int R, C, share, heads;
    float q_scale;
};

#define DELTA_GROUP_OF(RPT) ((RPT) >= 32 ? 4 : 8)

// The sum of x over the NG (4, 8 or 16) neighbouring lanes of an aligned group, in every lane of the group, by
// data-parallel-primitive moves inside a row of 16 lanes: neighbours, pairs, then the mirror image of a half row and
// of a row (the partial sums are by then the same in all lanes of a quad, of a half row).
template <int CTRL>
__device__ __forceinline__ float lanes_moved(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xF, 0xF, false));
}

template <int NG>
__device__ __forceinline__ float group_sum(float x) {
    x += lanes_moved<0xB1>(x);                   // quad_perm [1, 0, 3, 2]
    x += lanes_moved<0x4E>(x);                   // quad_perm [2, 3, 0, 1]
    if (NG >= 8) x += lanes_moved<0x141>(x);     // row_half_mirror
    if (NG >= 16) x += lanes_moved<0x140>(x);    // row_mirror
    return x;
}

// A wave a (segment, head, tile of COLS = 128 / NG columns); NG neighbouring lanes share two neighbouring columns, and
// lane l of them owns the rows l RPT + i, i < RPT, of the state in registers.  Rows of a segment are walked in order,
// GROUP at a time through LDS, the next group's loads in flight while this one is walked.  In LDS a lane's RPT
// coordinates of q and of k lie side by side (one wide read each), the lanes' runs PAD floats apart so that the reads of
// the sixteen lanes of a row fall into different banks.
template <int NG, int RPT>
__global__ void __launch_bounds__(64) delta_scan_kernel(DeltaArgs p) {
    constexpr int LPG = WAVE / NG, COLS = 2 * LPG, GROUP = DELTA_GROUP_OF(RPT), RP = NG * RPT;
    constexpr int PAD = RPT >= 4 ? 4 : 2, RUN = RPT + PAD, RPS = NG * RUN;     // floats of a lane's run, of a row in LDS
    __shared__ __attribute__((aligned(16))) float sq[GROUP * RPS], sk[GROUP * RPS];
    __shared__ float sg[GROUP], sb[GROUP], sv[GROUP * COLS];
    const int seg = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
    const int t0 = p.seg_start[seg], t1 = p.seg_start[seg + 1];
    if (t1 <= t0) return;
    const int pair = lane / NG, rg = lane % NG;
    const int c = blockIdx.z * COLS + 2 * pair;
    const bool ok0 = c < p.C, ok1 = c + 1 < p.C;
    const int c0 = ok0 ? c : p.C - 1, c1 = ok1 ? c + 1 : p.C - 1;
    const int R = p.R, C = p.C;
    float* state = p.state + (long long)p.state_slots[seg] * p.slot_stride + (size_t)head * R * C;
    float S0[RPT], S1[RPT];
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        const bool in = rg * RPT + i < R;
        S0[i] = in ? state[(size_t)(rg * RPT + i) * C + c0] : 0.f;
        S1[i] = in ? state[(size_t)(rg * RPT + i) * C + c1] : 0.f;
    }
    const float* qh = p.q + (size_t)(head / p.share) * R;
    const float* kh = p.k + (size_t)(head / p.share) * R;
    const float* vh = p.v + (size_t)head * C;
    constexpr int PF = GROUP * RP / WAVE, PV = (GROUP * COLS + WAVE - 1) / WAVE;
    static_assert(GROUP * RP % WAVE == 0, "a group's rows divide among the lanes");
    float fq[PF], fk[PF], fv[PV], fg = 0.f, fb = 0.f;
    auto fetch = [&](int tb) {
        const int last = t1 - 1;
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            const int idx = lane + WAVE * j, tt = idx / RP, r = idx % RP;
            const size_t t = (size_t)min(tb + tt, last);
            const bool in = r < R;
            const int rr = in ? r : 0;
            fk[j] = in ? kh[t * p.ldk + rr] : 0.f;
            fq[j] = in ? qh[t * p.ldq + rr] : 0.f;
        }
#pragma unroll
        for (int j = 0; j < PV; ++j) {
            const int idx = lane + WAVE * j, tt = min(idx / COLS, GROUP - 1), cc = blockIdx.z * COLS + idx % COLS;
            fv[j] = vh[(size_t)min(tb + tt, last) * p.ldv + min(cc, C - 1)];
        }
        if (lane < GROUP) {
            const size_t t = (size_t)min(tb + lane, last);
            fg = p.g[t * p.ldg + head];
            fb = p.b[t * p.ldb + head];
        }
    };
    fetch(t0);
    for (int tb = t0; tb < t1; tb += GROUP) {
        const int n = min(GROUP, t1 - tb);
        __syncthreads();                                   // (the walk before is over: LDS may be written)
#pragma unroll
        for (int j = 0; j < PF; ++j) {
            const int idx = lane + WAVE * j, tt = idx / RP, r = idx % RP;
            sk[tt * RPS + (r / RPT) * RUN + r % RPT] = fk[j];
            sq[tt * RPS + (r / RPT) * RUN + r % RPT] = fq[j];
        }
#pragma unroll
        for (int j = 0; j < PV; ++j)
            if (lane + WAVE * j < GROUP * COLS) sv[lane + WAVE * j] = fv[j];
        if (lane < GROUP) {
            sg[lane] = fg;
            sb[lane] = 1.0f / (1.0f + expf(-fb));
        }
        __syncthreads();
        if (tb + GROUP < t1) fetch(tb + GROUP);
#pragma unroll
        for (int tt = 0; tt < GROUP; ++tt) {
            if (tt >= n) break;                            // (uniform over the wave)
            float kc[RPT], qc[RPT];
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                kc[i] = sk[tt * RPS + rg * RUN + i];
                qc[i] = sq[tt * RPS + rg * RUN + i];
            }
            const float v0 = sv[tt * COLS + 2 * pair], v1 = sv[tt * COLS + 2 * pair + 1];
            const float g = sg[tt], beta = sb[tt];
            float sk0 = 0.f, sk1 = 0.f, sq0 = 0.f, sq1 = 0.f, kq = 0.f;
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                sk0 += S0[i] * kc[i];
                sk1 += S1[i] * kc[i];
                sq0 += S0[i] * qc[i];
                sq1 += S1[i] * qc[i];
                kq += kc[i] * qc[i];
            }
            sk0 = group_sum<NG>(sk0);
            sk1 = group_sum<NG>(sk1);
            sq0 = group_sum<NG>(sq0);
            sq1 = group_sum<NG>(sq1);
            kq = group_sum<NG>(kq);
            const float u0 = beta * (v0 - g * sk0), u1 = beta * (v1 - g * sk1);
#pragma unroll
            for (int i = 0; i < RPT; ++i) {
                S0[i] = g * S0[i] + kc[i] * u0;
                S1[i] = g * S1[i] + kc[i] * u1;
            }
            if (rg == 0) {
                float* o = p.out + (size_t)(tb + tt) * p.ldo + (size_t)head * C;
                if (ok0) o[c] = (g * sq0 + kq * u0) * p.q_scale;
                if (ok1) o[c + 1] = (g * sq1 + kq * u1) * p.q_scale;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < RPT; ++i) {
        if (rg * RPT + i >= R) continue;
        if (ok0) state[(size_t)(rg * RPT + i) * C + c] = S0[i];
        if (ok1) state[(size_t)(rg * RPT + i) * C + c + 1] = S1[i];
    }
}

template <int NG>
static int launch_delta_group(const DeltaArgs& p, int segments, hipStream_t stream) {
    constexpr int COLS = 2 * WAVE / NG;
    const int per = (p.R + NG - 1) / NG;                          // rows a lane
    const dim3 grid(segments, p.heads, (p.C + COLS - 1) / COLS);
    if (per <= 2) delta_scan_kernel<NG, 2><<<grid, 64, 0, stream>>>(p);
    else if (per <= 4) delta_scan_kernel<NG, 4><<<grid, 64, 0, stream>>>(p);
    else if (per <= 8) delta_scan_kernel<NG, 8><<<grid, 64, 0, stream>>>(p);
    else if (per <= 16) delta_scan_kernel<NG, 16><<<grid, 64, 0, stream>>>(p);
    else if (per <= 32) {
        // (32 rows of two columns a lane are what the registers hold; 16 lanes a column reach 256 rows with 16 each)
        if constexpr (NG <= 8) delta_scan_kernel<NG, 32><<<grid, 64, 0, stream>>>(p);
        else return (int)hipErrorInvalidValue;
    } else return (int)hipErrorInvalidValue;
    return CISR_LAUNCH_CHECK();
}

// cols: 8, 16 or 32 columns a wave (fewer columns are more waves for the same head, and shorter runs of the state);
// a lane holds at most 32 rows of its columns, so states of more than 128 rows need 16 columns or fewer.
extern "C" int cisr_delta_scan(const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                               const float* g, int ldg, const float* b, int ldb, float* out, int ldo,
                               float* state, long long slot_stride, const int* seg_start, const int* state_slots,
                               int segments, int heads, int R, int C, int share, float q_scale, int cols,
                               hipStream_t stream) {
    if (segments <= 0 || heads <= 0) return 0;
    if (R <= 0 || C <= 0 || share <= 0 || heads % share || heads > 65535 || (cols != 8 && cols != 16 && cols != 32) ||
        (C + cols - 1) / cols > 65535 || R > 256)
        return (int)hipErrorInvalidValue;
    DeltaArgs p{q, ldq, k, ldk, v, ldv, g, ldg, b, ldb, out, ldo, state, slot_stride, seg_start, state_slots, R, C, share, heads, q_scale};
    if (cols == 8) return launch_delta_group<16>(p, segments, stream);
    if (cols == 16) return launch_delta_group<8>(p, segments, stream);
    return launch_delta_group<4>(p, segments, stream);
}

// ------------------------------------------------------------------------------------------------ unit vectors
// x[t * ld + first + h * dim + i] <- x / sqrt(sum_i x^2 + eps) * scale, in place: a wave a (row, head).
__global__ void __launch_bounds__(256)
unit_heads_kernel(float* __restrict__ x, int ld, int first, int heads, int dim, float eps, float scale, int items) {
    const int item = blockIdx.x * 4 + threadIdx.x / WAVE, lane = threadIdx.x % WAVE;
    if (item >= items) return;
    float* row = x + (size_t)(item / heads) * ld + first + (size_t)(item % heads) * dim;
    float s = 0.f;
    for (int i = lane; i < dim; i += WAVE) s += row[i] * row[i];
    const float f = rsqrtf(wave_sum(s) + eps) * scale;
    for (int i = lane; i < dim; i += WAVE) row[i] *= f;
}

extern "C" int cisr_unit_heads(float* x, int ld, int first, int rows, int heads, int dim, float eps, float scale,
                               hipStream_t stream) {
    const long long items = (long long)rows * heads;
    if (items <= 0) return 0;
    if (dim <= 0 || first < 0 || first + heads * dim > ld || items > 0x7fffffff) return (int)hipErrorInvalidValue;
    unit_heads_kernel<<<(unsigned)((items + 3) / 4), 256, 0, stream>>>(x, ld, first, heads, dim, eps, scale, (int)items);
    return CISR_LAUNCH_CHECK();
}
