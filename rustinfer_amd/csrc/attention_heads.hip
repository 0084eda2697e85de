// What some attention mixers do to their projected rows, head by head, before the attention
// kernels see them (all arithmetic 32-bit, storage 32-bit or bfloat16):
//
//   head_norm_kv_write   queries and keys divided by their root mean square over the head, times a
//                        weight of the head's size shared by all heads, the query times a
//                        temperature that grows with the logarithm of its position; the query in
//                        place, the normed key and the value into the token's page;
//   latent_kv_write      attention through one latent vector a token: the first R features of the
//                        down projection are normed (c), the last r are one rotated key part for all
//                        heads; the page takes the key [c, rotated part] and the value c; the
//                        rotated part of every head's query goes to the tail of that head's
//                        absorbed query [R + r];
//   head_linear          out[t, h, :] = W_h x[t, h, :] for every head: the product that turns a
//                        head's unrotated query into the latent space (W_uk,h^T q) and the weighted
//                        sum of latents back into the head's value space (W_uv,h o).
//
// Cache layout as everywhere: keys [pages][Hkv][page][dk], values [pages][Hkv][dv][page].
#include "common.h"
#include <math.h>

namespace {

// ---------------------------------------------------------------------------
// Blocks (token, four heads): one wave a head (queries first, then keys); the blocks of a token's
// first heads also copy its values.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void head_norm_kv_write_kernel(
        T* __restrict__ q, int q_stride, const T* __restrict__ k, int k_stride, const T* __restrict__ v, int v_stride,
        int H, int Hkv, int dk, int dv, const float* __restrict__ qw, const float* __restrict__ kw, int do_norm, float eps,
        float temp_coef, int temp_every, const int* __restrict__ positions, const int* __restrict__ row_of_token,
        T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ table, int max_blocks, int page, int write_kv) {
    const int t = blockIdx.x;
    const int b = row_of_token[t];
    if (b < 0) return;                       // padding token
    const int pos = positions[t];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int blk = -1;
    if (write_kv) blk = table[(size_t)b * max_blocks + pos / page];
    const int slot = pos % page;
    const float temp = temp_every > 0 ? 1.f + temp_coef * logf((float)((pos + 1) / temp_every) + 1.f) : 1.f;
    const int units = H + (blk >= 0 ? Hkv : 0);
    for (int u = blockIdx.y * 4 + wave; u < units; u += 4 * gridDim.y) {
        const bool is_q = u < H;
        const int g = u - H;
        const T* src = is_q ? q + (size_t)t * q_stride + u * dk : k + (size_t)t * k_stride + g * dk;
        T* dst = is_q ? q + (size_t)t * q_stride + u * dk : kc + (((size_t)blk * Hkv + g) * page + slot) * dk;
        const float* w = is_q ? qw : kw;
        float f = is_q ? temp : 1.f;
        if (do_norm) {
            float ss = 0.f;
            for (int i = lane; i < dk; i += 64) { const float x = ld_f32(src + i); ss = fmaf(x, x, ss); }
            ss = wave_sum(ss);
            f *= 1.f / sqrtf(ss / (float)dk + eps);
        }
        for (int i = lane; i < dk; i += 64) {
            const float x = ld_f32(src + i);
            st_f32(dst + i, x * f * (w ? w[i] : 1.f));
        }
    }
    if (blk < 0) return;
    const T* vrow = v + (size_t)t * v_stride;
    for (int idx = blockIdx.y * 256 + threadIdx.x; idx < Hkv * dv; idx += 256 * gridDim.y) {
        const int g = idx / dv, dd = idx - g * dv;
        vc[(((size_t)blk * Hkv + g) * dv + dd) * page + slot] = vrow[idx];
    }
}

// ---------------------------------------------------------------------------
// One block a token.  q [T][H (d + r)]: a head's unrotated features, then its r rotated ones, of which
// the first `rot` are turned (feature i with i + rot/2).  down [T][R + r].  q_abs [T][H (R + r)].
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void latent_kv_write_kernel(
        const T* __restrict__ q, int q_stride, const T* __restrict__ down, int down_stride, T* __restrict__ q_abs, int qa_stride,
        int H, int d, int r, int R, int rot, const float* __restrict__ cw, float eps,
        const float* __restrict__ cos_t, const float* __restrict__ sin_t,
        const int* __restrict__ positions, const int* __restrict__ row_of_token,
        T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ table, int max_blocks, int page, int write_kv) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int b = row_of_token[t];
    if (b < 0) return;                       // padding token
    const int pos = positions[t];
    const int half = rot >> 1;
    const bool rotate = cos_t != nullptr && half > 0;
    const float* cs = rotate ? cos_t + (size_t)pos * half : nullptr;
    const float* sn = rotate ? sin_t + (size_t)pos * half : nullptr;
    auto turned = [&](const T* part, int j) -> float {      // feature j of a rotated part after the turn
        if (rotate && j < half) return ld_f32(part + j) * cs[j] - ld_f32(part + j + half) * sn[j];
        if (rotate && j < rot) return ld_f32(part + j) * cs[j - half] + ld_f32(part + j - half) * sn[j - half];
        return ld_f32(part + j);
    };
    const T* qrow = q + (size_t)t * q_stride;
    T* qa = q_abs + (size_t)t * qa_stride;
    for (int idx = threadIdx.x; idx < H * r; idx += 256) {
        const int h = idx / r, j = idx - h * r;
        st_f32(qa + h * (R + r) + R + j, turned(qrow + h * (d + r) + d, j));
    }
    if (!write_kv) return;
    const int blk = table[(size_t)b * max_blocks + pos / page];
    if (blk < 0) return;                     // (uniform over the block)
    const int slot = pos % page;
    const T* drow = down + (size_t)t * down_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < R; i += 256) { const float x = ld_f32(drow + i); ss = fmaf(x, x, ss); }
    ss = block_sum(ss, red);
    const float rs = 1.f / sqrtf(ss / (float)R + eps);
    T* krow = kc + ((size_t)blk * page + slot) * (R + r);
    for (int i = threadIdx.x; i < R; i += 256) {
        const float c = ld_f32(drow + i) * rs * (cw ? cw[i] : 1.f);
        st_f32(krow + i, c);
        st_f32(vc + ((size_t)blk * R + i) * page + slot, c);
    }
    for (int j = threadIdx.x; j < r; j += 256) st_f32(krow + R + j, turned(drow + R, j));
}

// ---------------------------------------------------------------------------
// out[t][h * out_head + n] = sum_k x[t][h * x_head + k] * w[(h * N + n) * K + k],  n < N, k < K.
// A block of 256 threads owns 64 tokens x 64 outputs of one head; K goes by in steps of 16 through
// LDS; a thread sums a 4 x 4 patch in 32-bit, in the order of k.
// ---------------------------------------------------------------------------
constexpr int HL_T = 64, HL_N = 64, HL_K = 16;

template <typename T>
__global__ __launch_bounds__(256) void head_linear_kernel(
        const T* __restrict__ x, int x_stride, int x_head, const T* __restrict__ w, T* __restrict__ out, int out_stride,
        int out_head, int Tn, int N, int K) {
    __shared__ float xs[HL_K][HL_T + 4];
    __shared__ float ws[HL_K][HL_N + 4];
    const int h = blockIdx.z, t0 = blockIdx.x * HL_T, n0 = blockIdx.y * HL_N;
    const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;           // outputs 4 tx.., tokens 4 ty..
    const T* wh = w + (size_t)h * N * K;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += HL_K) {
        for (int e = threadIdx.x; e < HL_T * HL_K; e += 256) {
            const int kk = e % HL_K, tt = e / HL_K;
            const int t = t0 + tt, k = k0 + kk;
            xs[kk][tt] = (t < Tn && k < K) ? ld_f32(x + (size_t)t * x_stride + h * x_head + k) : 0.f;
        }
        for (int e = threadIdx.x; e < HL_N * HL_K; e += 256) {
            const int kk = e % HL_K, nn = e / HL_K;
            const int n = n0 + nn, k = k0 + kk;
            ws[kk][nn] = (n < N && k < K) ? ld_f32(wh + (size_t)n * K + k) : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < HL_K; ++kk) {
            const float4 xv = *reinterpret_cast<const float4*>(&xs[kk][4 * ty]);
            const float4 wv = *reinterpret_cast<const float4*>(&ws[kk][4 * tx]);
            const float xa[4] = {xv.x, xv.y, xv.z, xv.w}, wa[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(xa[i], wa[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int t = t0 + 4 * ty + i;
        if (t >= Tn) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int n = n0 + 4 * tx + j;
            if (n < N) st_f32(out + (size_t)t * out_stride + h * out_head + n, acc[i][j]);
        }
    }
}

// The same product for a step of few tokens (up to HLF_T): no staging.  Eight lanes share an output
// and divide K between them in pieces of 16 bytes (VEC: operands aligned for that; else element by
// element), each summing all tokens' terms of its pieces; a block owns 32 outputs of one head.  The
// sums of a token are added in a fixed order whatever else the step holds.
constexpr int HLF_T = 16;

__device__ __forceinline__ void hl_ld16(const float* p, float* f) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    f[0] = v.x; f[1] = v.y; f[2] = v.z; f[3] = v.w;
}
__device__ __forceinline__ void hl_ld16(const bf16_t* p, float* f) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
    f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
    f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
    f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

template <typename T, bool VEC>
__global__ __launch_bounds__(256) void head_linear_few_kernel(
        const T* __restrict__ x, int x_stride, int x_head, const T* __restrict__ w, T* __restrict__ out, int out_stride,
        int out_head, int Tn, int N, int K) {
    constexpr int VL = VEC ? 16 / (int)sizeof(T) : 1;
    const int h = blockIdx.y, part = threadIdx.x & 7, n = blockIdx.x * 32 + (threadIdx.x >> 3);
    const bool live = n < N;
    const T* wr = w + ((size_t)h * N + (live ? n : 0)) * K;
    const T* xh = x + (size_t)h * x_head;
    float acc[HLF_T];
#pragma unroll
    for (int t = 0; t < HLF_T; ++t) acc[t] = 0.f;
    for (int k = part * VL; k < K; k += 8 * VL) {
        float wv[VL];
        if (VEC) hl_ld16(wr + k, wv); else wv[0] = ld_f32(wr + k);
#pragma unroll
        for (int t = 0; t < HLF_T; ++t) {
            if (t >= Tn) break;
            float xv[VL];
            if (VEC) hl_ld16(xh + (size_t)t * x_stride + k, xv); else xv[0] = ld_f32(xh + (size_t)t * x_stride + k);
#pragma unroll
            for (int u = 0; u < VL; ++u) acc[t] = fmaf(xv[u], wv[u], acc[t]);
        }
    }
#pragma unroll
    for (int t = 0; t < HLF_T; ++t) {
        if (t >= Tn) break;
        float v = acc[t];
#pragma unroll
        for (int o = 4; o > 0; o >>= 1) v += __shfl_xor(v, o, 8);
        if (part == 0 && live) st_f32(out + (size_t)t * out_stride + h * out_head + n, v);
    }
}

}  // namespace

// q [T][>= H dk] is normed in place; k [T][>= Hkv dk], v [T][>= Hkv dv] go to the token's page
// (write_kv; a layer that reads another layer's cache has none).  qw, kw: 32-bit weights of dk
// entries or null; do_norm 0: no division by the root mean square (weights and temperature only).
// temp_every > 0: the query at position p is multiplied by 1 + temp_coef ln(floor((p + 1) / temp_every) + 1).
extern "C" int ri_head_norm_kv_write(
        void* q, int q_stride, const void* k, int k_stride, const void* v, int v_stride, int dtype, int T,
        int H, int Hkv, int dk, int dv, const float* qw, const float* kw, int do_norm, float eps,
        float temp_coef, int temp_every, const int* positions, const int* row_of_token,
        void* kc, void* vc, int num_pages, const int* table, int max_blocks, int page, int write_kv, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && Hkv > 0 && dk > 0 && dv > 0 && page > 0, "ri_head_norm_kv_write: bad sizes");
    RI_REQUIRE(q_stride >= H * dk, "ri_head_norm_kv_write: query row stride %d too small", q_stride);
    RI_REQUIRE(!do_norm || eps > 0.f, "ri_head_norm_kv_write: eps must be > 0");
    if (write_kv) RI_REQUIRE(k && v && kc && vc && table && max_blocks > 0 && num_pages > 0 && k_stride >= Hkv * dk && v_stride >= Hkv * dv,
                             "ri_head_norm_kv_write: no keys, values or cache given, or their row strides too small");
    if (T == 0) return 0;
    RI_REQUIRE(q && positions && row_of_token, "ri_head_norm_kv_write: null pointer");
    // a step of few tokens: a block for every four heads, so that no wave walks a chain of heads
    const int by = T <= 256 ? min((H + Hkv + 3) / 4, 64) : 1;
    const dim3 grid(T, by);
    if (dtype == RI_F32)
        head_norm_kv_write_kernel<float><<<grid, 256, 0, stream>>>((float*)q, q_stride, (const float*)k, k_stride, (const float*)v, v_stride, H, Hkv, dk, dv, qw, kw, do_norm, eps, temp_coef, temp_every, positions, row_of_token, (float*)kc, (float*)vc, table, max_blocks, page, write_kv);
    else if (dtype == RI_BF16)
        head_norm_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)q, q_stride, (const bf16_t*)k, k_stride, (const bf16_t*)v, v_stride, H, Hkv, dk, dv, qw, kw, do_norm, eps, temp_coef, temp_every, positions, row_of_token, (bf16_t*)kc, (bf16_t*)vc, table, max_blocks, page, write_kv);
    else
        return ri_fail("ri_head_norm_kv_write: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_head_norm_kv_write");
    return 0;
}

// The cache belongs to one key/value head with keys of R + r features and values of R.
extern "C" int ri_latent_kv_write(
        const void* q, int q_stride, const void* down, int down_stride, void* q_abs, int qa_stride, int dtype, int T,
        int H, int d, int r, int R, int rot, const float* cw, float eps, const float* cos_t, const float* sin_t, int table_rows,
        const int* positions, const int* row_of_token, void* kc, void* vc, int num_pages,
        const int* table, int max_blocks, int page, int write_kv, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && d >= 0 && r >= 0 && R > 0 && page > 0, "ri_latent_kv_write: bad sizes");
    RI_REQUIRE(q_stride >= H * (d + r) && qa_stride >= H * (R + r) && down_stride >= R + r, "ri_latent_kv_write: row strides too small");
    RI_REQUIRE(eps > 0.f, "ri_latent_kv_write: eps must be > 0");
    if (cos_t) RI_REQUIRE(rot > 0 && rot % 2 == 0 && rot <= r && sin_t && table_rows > 0, "ri_latent_kv_write: rot %d must be even and within the rotated part %d", rot, r);
    if (write_kv) RI_REQUIRE(kc && vc && table && max_blocks > 0 && num_pages > 0, "ri_latent_kv_write: no cache given");
    if (T == 0) return 0;
    RI_REQUIRE(q && down && q_abs && positions && row_of_token, "ri_latent_kv_write: null pointer");
    if (dtype == RI_F32)
        latent_kv_write_kernel<float><<<T, 256, 0, stream>>>((const float*)q, q_stride, (const float*)down, down_stride, (float*)q_abs, qa_stride, H, d, r, R, rot, cw, eps, cos_t, sin_t, positions, row_of_token, (float*)kc, (float*)vc, table, max_blocks, page, write_kv);
    else if (dtype == RI_BF16)
        latent_kv_write_kernel<bf16_t><<<T, 256, 0, stream>>>((const bf16_t*)q, q_stride, (const bf16_t*)down, down_stride, (bf16_t*)q_abs, qa_stride, H, d, r, R, rot, cw, eps, cos_t, sin_t, positions, row_of_token, (bf16_t*)kc, (bf16_t*)vc, table, max_blocks, page, write_kv);
    else
        return ri_fail("ri_latent_kv_write: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_latent_kv_write");
    return 0;
}

// x [T][x_stride], head h at column h * x_head; w [H][N][K] contiguous; out [T][out_stride], head h
// at column h * out_head.
extern "C" int ri_head_linear(const void* x, int x_stride, int x_head, const void* w, void* out, int out_stride, int out_head,
                              int dtype, int T, int H, int N, int K, hipStream_t stream) {
    RI_REQUIRE(T >= 0 && H > 0 && N > 0 && K > 0, "ri_head_linear: bad sizes T=%d H=%d N=%d K=%d", T, H, N, K);
    RI_REQUIRE(x_head >= 0 && out_head >= 0 && x_stride >= (H - 1) * x_head + K && out_stride >= (H - 1) * out_head + N,
               "ri_head_linear: row strides too small");
    if (T == 0) return 0;
    RI_REQUIRE(x && w && out, "ri_head_linear: null pointer");
    RI_REQUIRE(H <= 65535 && (N + HL_N - 1) / HL_N <= 65535, "ri_head_linear: too many heads or outputs for the grid");
    if (T <= HLF_T) {
        const dim3 few((N + 31) / 32, H);
        const int vl = dtype == RI_F32 ? 4 : 8;
        const bool vec = K % vl == 0 && x_stride % vl == 0 && x_head % vl == 0 && (uintptr_t)x % 16 == 0 && (uintptr_t)w % 16 == 0;
#define RI_HLF(TT, VV) head_linear_few_kernel<TT, VV><<<few, 256, 0, stream>>>((const TT*)x, x_stride, x_head, (const TT*)w, (TT*)out, out_stride, out_head, T, N, K)
        if (dtype == RI_F32) { if (vec) RI_HLF(float, true); else RI_HLF(float, false); }
        else if (dtype == RI_BF16) { if (vec) RI_HLF(bf16_t, true); else RI_HLF(bf16_t, false); }
        else
            return ri_fail("ri_head_linear: unknown dtype %d", dtype);
#undef RI_HLF
        RI_LAUNCHED("ri_head_linear");
        return 0;
    }
    const dim3 grid((T + HL_T - 1) / HL_T, (N + HL_N - 1) / HL_N, H);
    if (dtype == RI_F32)
        head_linear_kernel<float><<<grid, 256, 0, stream>>>((const float*)x, x_stride, x_head, (const float*)w, (float*)out, out_stride, out_head, T, N, K);
    else if (dtype == RI_BF16)
        head_linear_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)x, x_stride, x_head, (const bf16_t*)w, (bf16_t*)out, out_stride, out_head, T, N, K);
    else
        return ri_fail("ri_head_linear: unknown dtype %d", dtype);
    RI_LAUNCHED("ri_head_linear");
    return 0;
}
