// Mixers that carry a matrix of state from token to token instead of a cache of keys:
//
//   S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,      o_t = S_t^T r_t
//
// per head, S of [dk][dv] 32-bit floats in the request's state slot.  Two forms:
//   decay form:  w_t = one constant per head, no second term (a = 0); r, k, v may pass through silu
//                (linear attention with a fixed decay);
//   delta form:  u_t = k_t / sqrt(|k_t|^2 + unit_eps),  w_t = exp(-c * sigmoid(wl_t + w0)),
//                a_t = sigmoid(al_t + ab), all per key channel (a generalized delta rule: the
//                state forgets by w and gives up what it held along u at the rate a).
// Both terms of the delta form read the old state.  Everything after the projections is 32-bit.
//
// One kernel walks a request's tokens of the step in order; a step of single tokens is the same
// walk of one token.  A thread keeps 32 key rows of one value column in registers; the P threads
// that share a column (P = the power of two with 32 P >= dk) sit in one wave, 64 / P lanes apart,
// and add their partial dot products with lane exchanges.  The vectors of a stretch of eight
// tokens are brought into LDS, activated, by the whole block; the walk then reads them as
// broadcasts.  What a token adds up, and in which order, does not depend on how the request was
// cut into steps, so the state and the outputs have the same bits for every cut.
// A block holds NW waves (64 NW / P columns); with few (request, head) pairs a wave a block, so
// that the chip has blocks enough.
#include "common.h"
#include <math.h>

namespace {

constexpr int SC_R = 32;         // key rows a thread
constexpr int SC_CH = 8;         // tokens a stretch

struct ScanArgs {
    const void *r, *k, *v, *wl, *al;
    int r_stride, k_stride, v_stride, wl_stride, al_stride;
    const float *w0, *ab, *decay;
    float* state;
    float* out;
    int out_stride;
    const int *cu_q, *q_start, *slots;
    int H, dk, dv, P, silu_in;
    float unit_eps, decay_c;
};

__device__ __forceinline__ float sigmoidf_(float z) { return 1.f / (1.f + expf(-z)); }
__device__ __forceinline__ float siluf_(float z) { return z / (1.f + expf(-z)); }

template <typename T, bool DELTA, int NW>
__global__ __launch_bounds__(NW * 64) void linear_scan_kernel(const ScanArgs a) {
    extern __shared__ __align__(16) float lds[];
    const int P = a.P, DKP = P * SC_R, dk = a.dk, dv = a.dv, H = a.H;
    const int CW = 64 / P, CPB = NW * CW;
    float* rs = lds;                                   // [SC_CH][DKP]
    float* ks = rs + SC_CH * DKP;
    float* us = ks + SC_CH * DKP;                      // the delta form's three
    float* aus = us + SC_CH * DKP;
    float* ws = aus + SC_CH * DKP;
    float* vs = DELTA ? ws + SC_CH * DKP : us;         // [SC_CH][CPB]
    const int b = blockIdx.z, h = blockIdx.y;
    const int t_lo = a.cu_q[b], n = a.cu_q[b + 1] - t_lo;
    if (n <= 0) return;                                // a row without tokens (padding of a captured shape)
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int pl = lane / CW, cl = lane - pl * CW;
    const int jc = wave * CW + cl, j = blockIdx.x * CPB + jc;
    const bool col_ok = j < dv;
    float* Sg = a.state + ((size_t)a.slots[b] * H + h) * (size_t)dk * dv;
    const bool fresh = a.q_start[b] == 0;              // a request's first tokens start from nothing
    float S[SC_R];
#pragma unroll
    for (int ii = 0; ii < SC_R; ++ii) {
        const int i = pl * SC_R + ii;
        S[ii] = (!fresh && col_ok && i < dk) ? Sg[(size_t)i * dv + j] : 0.f;
    }
    const float dec = DELTA ? 0.f : a.decay[h];
    const T* rp = (const T*)a.r; const T* kp = (const T*)a.k; const T* vp = (const T*)a.v;
    const T* wlp = (const T*)a.wl; const T* alp = (const T*)a.al;
    for (int c0 = 0; c0 < n; c0 += SC_CH) {
        const int nc = min(SC_CH, n - c0);
        __syncthreads();                               // the last stretch has been walked
        for (int tt = wave; tt < nc; tt += NW) {
            const size_t t = (size_t)(t_lo + c0 + tt);
            if (DELTA) {
                float kk[4], ssq = 0.f;                // DKP / 64 <= 4 values a lane
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = e * 64 + lane;
                    kk[e] = (i < dk) ? ld_f32(kp + t * a.k_stride + h * dk + i) : 0.f;
                    ssq = fmaf(kk[e], kk[e], ssq);
                }
                ssq = wave_sum(ssq);
                const float inv = 1.f / sqrtf(ssq + a.unit_eps);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int i = e * 64 + lane;
                    if (i >= DKP) continue;
                    float r = 0.f, u = 0.f, au = 0.f, w = 0.f;
                    if (i < dk) {
                        const int c = h * dk + i;
                        r = ld_f32(rp + t * a.r_stride + c);
                        u = kk[e] * inv;
                        au = sigmoidf_(ld_f32(alp + t * a.al_stride + c) + a.ab[c]) * u;
                        w = expf(-a.decay_c * sigmoidf_(ld_f32(wlp + t * a.wl_stride + c) + a.w0[c]));
                    }
                    rs[tt * DKP + i] = r; ks[tt * DKP + i] = kk[e];
                    us[tt * DKP + i] = u; aus[tt * DKP + i] = au; ws[tt * DKP + i] = w;
                }
            } else {
                for (int i = lane; i < DKP; i += 64) {
                    float r = 0.f, k = 0.f;
                    if (i < dk) {
                        r = ld_f32(rp + t * a.r_stride + h * dk + i);
                        k = ld_f32(kp + t * a.k_stride + h * dk + i);
                        if (a.silu_in) { r = siluf_(r); k = siluf_(k); }
                    }
                    rs[tt * DKP + i] = r; ks[tt * DKP + i] = k;
                }
            }
        }
        for (int e = tid; e < nc * CPB; e += NW * 64) {
            const int tt = e / CPB, c = e - tt * CPB, jj = blockIdx.x * CPB + c;
            float v = 0.f;
            if (jj < dv) {
                v = ld_f32(vp + (size_t)(t_lo + c0 + tt) * a.v_stride + h * dv + jj);
                if (!DELTA && a.silu_in) v = siluf_(v);
            }
            vs[e] = v;
        }
        __syncthreads();
        for (int tt = 0; tt < nc; ++tt) {
            const float vv = vs[tt * CPB + jc];
            const int base = tt * DKP + pl * SC_R;
            if (DELTA) {
                float dot = 0.f;
#pragma unroll
                for (int ii = 0; ii < SC_R; ii += 4) {
                    const float4 u4 = *reinterpret_cast<const float4*>(us + base + ii);
                    dot = fmaf(u4.x, S[ii], dot); dot = fmaf(u4.y, S[ii + 1], dot);
                    dot = fmaf(u4.z, S[ii + 2], dot); dot = fmaf(u4.w, S[ii + 3], dot);
                }
                for (int o = CW; o < 64; o <<= 1) dot += __shfl_xor(dot, o, 64);
#pragma unroll
                for (int ii = 0; ii < SC_R; ii += 4) {
                    const float4 w4 = *reinterpret_cast<const float4*>(ws + base + ii);
                    const float4 a4 = *reinterpret_cast<const float4*>(aus + base + ii);
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + base + ii);
                    S[ii] = fmaf(w4.x, S[ii], fmaf(-a4.x, dot, k4.x * vv));
                    S[ii + 1] = fmaf(w4.y, S[ii + 1], fmaf(-a4.y, dot, k4.y * vv));
                    S[ii + 2] = fmaf(w4.z, S[ii + 2], fmaf(-a4.z, dot, k4.z * vv));
                    S[ii + 3] = fmaf(w4.w, S[ii + 3], fmaf(-a4.w, dot, k4.w * vv));
                }
            } else {
#pragma unroll
                for (int ii = 0; ii < SC_R; ii += 4) {
                    const float4 k4 = *reinterpret_cast<const float4*>(ks + base + ii);
                    S[ii] = fmaf(dec, S[ii], k4.x * vv); S[ii + 1] = fmaf(dec, S[ii + 1], k4.y * vv);
                    S[ii + 2] = fmaf(dec, S[ii + 2], k4.z * vv); S[ii + 3] = fmaf(dec, S[ii + 3], k4.w * vv);
                }
            }
            float o = 0.f;
#pragma unroll
            for (int ii = 0; ii < SC_R; ii += 4) {
                const float4 r4 = *reinterpret_cast<const float4*>(rs + base + ii);
                o = fmaf(r4.x, S[ii], o); o = fmaf(r4.y, S[ii + 1], o);
                o = fmaf(r4.z, S[ii + 2], o); o = fmaf(r4.w, S[ii + 3], o);
            }
            for (int s = CW; s < 64; s <<= 1) o += __shfl_xor(o, s, 64);
            if (pl == 0 && col_ok) a.out[(size_t)(t_lo + c0 + tt) * a.out_stride + h * dv + j] = o;
        }
    }
#pragma unroll
    for (int ii = 0; ii < SC_R; ++ii) {
        const int i = pl * SC_R + ii;
        if (col_ok && i < dk) Sg[(size_t)i * dv + j] = S[ii];
    }
}

template <typename T, bool DELTA>
int launch_scan(const ScanArgs& a, int num_rows, hipStream_t stream) {
    const int P = a.P, DKP = P * SC_R;
    // four waves a block unless that leaves most of the chip without a block
    const int cols4 = 4 * (64 / P);
    const long blocks4 = (long)((a.dv + cols4 - 1) / cols4) * a.H * num_rows;
    const int NW = blocks4 >= 256 ? 4 : 1;
    const int CPB = NW * (64 / P);
    const size_t lds = sizeof(float) * ((DELTA ? 5 : 2) * SC_CH * DKP + SC_CH * CPB);
    dim3 grid((a.dv + CPB - 1) / CPB, a.H, num_rows);
    if (NW == 4) linear_scan_kernel<T, DELTA, 4><<<grid, 256, lds, stream>>>(a);
    else linear_scan_kernel<T, DELTA, 1><<<grid, 64, lds, stream>>>(a);
    return 0;
}

}  // namespace

// The walk for the tokens of a step.  r, k [T, >= H dk], v [T, >= H dv] are columns of the
// projections (any row stride), in `dtype`; wl, al, w0, ab go with the delta form (delta != 0),
// decay [H] with the decay form.  state [slots][H][dk][dv] and out [T][out_stride >= H dv] are
// 32-bit.  A row whose q_start is 0 starts from a state of zeros (its slot is overwritten).
extern "C" int ri_linear_scan(
        const void* r, int r_stride, const void* k, int k_stride, const void* v, int v_stride,
        const void* wl, int wl_stride, const void* al, int al_stride, int dtype,
        const float* w0, const float* ab, const float* decay, int delta, int silu_in,
        float unit_eps, float decay_c, float* state, int num_slots, float* out, int out_stride,
        const int* cu_q, const int* q_start, const int* slots, int num_rows, int T,
        int H, int dk, int dv, hipStream_t stream) {
    RI_REQUIRE(H > 0 && dk > 0 && dv > 0 && dk <= 256, "ri_linear_scan: bad sizes H=%d dk=%d dv=%d (dk <= 256)", H, dk, dv);
    RI_REQUIRE(num_rows >= 0 && T >= 0 && num_slots > 0, "ri_linear_scan: bad counts");
    RI_REQUIRE(r_stride >= H * dk && k_stride >= H * dk && v_stride >= H * dv && out_stride >= H * dv,
               "ri_linear_scan: row strides too small");
    if (num_rows == 0 || T == 0) return 0;
    RI_REQUIRE(r && k && v && state && out && cu_q && q_start && slots, "ri_linear_scan: null pointer");
    RI_REQUIRE(H <= 65535 && num_rows <= 65535, "ri_linear_scan: too many heads or rows for the grid");
    if (delta) RI_REQUIRE(wl && al && w0 && ab && wl_stride >= H * dk && al_stride >= H * dk, "ri_linear_scan: the delta form needs wl, al, w0, ab");
    else RI_REQUIRE(decay, "ri_linear_scan: the decay form needs a decay for each head");
    int P = 1;
    while (P * SC_R < dk) P *= 2;
    ScanArgs a;
    a.r = r; a.k = k; a.v = v; a.wl = wl; a.al = al;
    a.r_stride = r_stride; a.k_stride = k_stride; a.v_stride = v_stride; a.wl_stride = wl_stride; a.al_stride = al_stride;
    a.w0 = w0; a.ab = ab; a.decay = decay; a.state = state; a.out = out; a.out_stride = out_stride;
    a.cu_q = cu_q; a.q_start = q_start; a.slots = slots;
    a.H = H; a.dk = dk; a.dv = dv; a.P = P; a.silu_in = silu_in; a.unit_eps = unit_eps; a.decay_c = decay_c;
    if (dtype == RI_F32) { if (delta) launch_scan<float, true>(a, num_rows, stream); else launch_scan<float, false>(a, num_rows, stream); }
    else if (dtype == RI_BF16) { if (delta) launch_scan<bf16_t, true>(a, num_rows, stream); else launch_scan<bf16_t, false>(a, num_rows, stream); }
    else return ri_fail("ri_linear_scan: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_linear_scan");
    return 0;
}

// ---------------------------------------------------------------------------
// y = o / sqrt(mean_group(o^2) + eps) * w * sigmoid(gate): the norm over groups of `group`
// consecutive features (all of a row, or a head) that follows the walk, with the output gate.
// o is 32-bit; gate and out are activations of `dtype` with row strides; w has n entries.
// A wave a group.
// ---------------------------------------------------------------------------
namespace {
template <typename T, typename TW>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(
        const float* __restrict__ o, int o_stride, int n, int group, const TW* __restrict__ w,
        const T* __restrict__ gate, int gate_stride, T* __restrict__ out, int out_stride, float eps) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const float* orow = o + (size_t)t * o_stride;
    for (int g0 = wave * group; g0 < n; g0 += nw * group) {
        float ss = 0.f;
        for (int i = lane; i < group; i += 64) { const float x = orow[g0 + i]; ss = fmaf(x, x, ss); }
        ss = wave_sum(ss);
        const float inv = 1.f / sqrtf(ss / (float)group + eps);
        for (int i = lane; i < group; i += 64) {
            const int c = g0 + i;
            float y = orow[c] * inv * ld_f32(w + c);
            if (gate) y *= sigmoidf_(ld_f32(gate + (size_t)t * gate_stride + c));
            st_f32(out + (size_t)t * out_stride + c, y);
        }
    }
}
}  // namespace

extern "C" int ri_gated_group_norm(const float* o, int o_stride, int T, int n, int group, const void* w, int w_dtype,
                                   const void* gate, int gate_stride, void* out, int out_stride, int dtype,
                                   float eps, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && n > 0 && group > 0 && n % group == 0, "ri_gated_group_norm: %d features do not split into groups of %d", n, group);
    RI_REQUIRE(o_stride >= n && out_stride >= n && (!gate || gate_stride >= n), "ri_gated_group_norm: row strides too small");
    if (T == 0) return 0;
    RI_REQUIRE(o && w && out, "ri_gated_group_norm: null pointer");
    const int block = 64 * min(4, n / group);
#define RI_GGN(TT, TW) gated_group_norm_kernel<TT, TW><<<T, block, 0, stream>>>(o, o_stride, n, group, (const TW*)w, (const TT*)gate, gate_stride, (TT*)out, out_stride, eps)
    if (dtype == RI_F32 && w_dtype == RI_F32) RI_GGN(float, float);
    else if (dtype == RI_BF16 && w_dtype == RI_F32) RI_GGN(bf16_t, float);
    else if (dtype == RI_BF16 && w_dtype == RI_BF16) RI_GGN(bf16_t, bf16_t);
    else return ri_fail("ri_gated_group_norm: dtypes %d / %d not taken", dtype, w_dtype);
#undef RI_GGN
    RI_LAUNCHED("ri_gated_group_norm");
    return 0;
}
