// RMSNorm / fused (split-K reduce +) residual + RMSNorm for gfx950.
//
// Replaces: src/turbomind/kernels/norm/rms_norm.cu:21-138 (invokeRMSNorm) and
//           :286-362,423-466 (invokeResidualBiasRMSNorm).
// Arithmetic (rms_norm_utils.cuh:6-15): r = h(r + hcur) [then h(r + bias)];
//   inv = rsqrtf(sum f32(r)^2 / H + eps);  y = h( h(f32(r) * inv) * w ).
// One workgroup per token row; 16-byte vector accesses; the row lives in registers between the two
// passes (norm_row.h).  Latency-bound (tiny): the point is fusing the split-K reduce of the
// preceding row-parallel GEMM so that no extra launch / HBM round trip is spent on it.
#include "tm_common.h"
#include "tm_kernels.h"
#include "norm_row.h"

namespace tmk {

template<int MODE, bool HAS_BIAS, int NV>
__global__ __launch_bounds__(kNormMaxThreads) void rmsnorm_kernel(half_t* __restrict__ y,
                                                                  half_t* __restrict__ resid,
                                                                  const half_t* __restrict__ hidden,
                                                                  const float* __restrict__ partial,
                                                                  int           splits,
                                                                  const half_t* __restrict__ bias,
                                                                  const half_t* __restrict__ weight,
                                                                  float eps,
                                                                  int   M,
                                                                  int   H,
                                                                  uint64_t* dbg)
{
    __shared__ float red[8];
    if (dbg && threadIdx.x == 0) {
        dbg[blockIdx.x * 8 + 0] = __builtin_amdgcn_s_memrealtime();
        dbg[blockIdx.x * 8 + 4] = ((uint64_t)__builtin_amdgcn_s_getreg(20 | (31 << 11)) << 32) | (uint32_t)__builtin_amdgcn_s_getreg(4 | (31 << 11));
    }
    norm_row<MODE, HAS_BIAS, NV>(y, resid, hidden, partial, splits, bias, weight, eps, M, H, blockIdx.x, threadIdx.x, blockDim.x, red);
    if (dbg && threadIdx.x == 0) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        dbg[blockIdx.x * 8 + 3] = __builtin_amdgcn_s_memrealtime();
    }
}

int launch_rmsnorm(half_t* y, const half_t* x, const half_t* w, float eps, int M, int H, hipStream_t st)
{
    TM_REQUIRE(H % 8 == 0 && H <= kNormMaxThreads * kNormMaxVec * 8, "rmsnorm: H must be a multiple of 8 and <= 8192");
    if (M == 0) {
        return 0;
    }
    int threads, nv;
    norm_geometry(H, &threads, &nv);
    uint64_t* const dbg = gemm_trace_for((size_t)M, "norm", M, 1, 1);
    if (nv == 1) {
        rmsnorm_kernel<0, false, 1><<<M, threads, 0, st>>>(y, nullptr, x, nullptr, 0, nullptr, w, eps, M, H, dbg);
    }
    else {
        rmsnorm_kernel<0, false, 2><<<M, threads, 0, st>>>(y, nullptr, x, nullptr, 0, nullptr, w, eps, M, H, dbg);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

int launch_residual_rmsnorm(half_t*       y,
                            half_t*       resid,
                            const half_t* hidden,
                            const float*  partial,
                            int           splits,
                            const half_t* bias,
                            const half_t* w,
                            float         eps,
                            int           M,
                            int           H,
                            hipStream_t   st)
{
    TM_REQUIRE(H % 8 == 0 && H <= kNormMaxThreads * kNormMaxVec * 8, "rmsnorm: H must be a multiple of 8 and <= 8192");
    TM_REQUIRE((hidden != nullptr) != (partial != nullptr), "exactly one of hidden / partial");
    TM_REQUIRE(!partial || splits >= 1, "splits >= 1");
    if (M == 0) {
        return 0;
    }
    int threads, nv;
    norm_geometry(H, &threads, &nv);
    uint64_t* const dbg = gemm_trace_for((size_t)M, partial ? "reduce_norm" : "resid_norm", M, 1, 1);
#define TM_NORM_LAUNCH(MODE, BIAS)                                                                                    \
    if (nv == 1) {                                                                                                    \
        rmsnorm_kernel<MODE, BIAS, 1><<<M, threads, 0, st>>>(y, resid, hidden, partial, splits, bias, w, eps, M, H, dbg);  \
    }                                                                                                                 \
    else {                                                                                                            \
        rmsnorm_kernel<MODE, BIAS, 2><<<M, threads, 0, st>>>(y, resid, hidden, partial, splits, bias, w, eps, M, H, dbg);  \
    }
    if (partial) {
        if (bias) {
            TM_NORM_LAUNCH(2, true)
        }
        else {
            TM_NORM_LAUNCH(2, false)
        }
    }
    else {
        if (bias) {
            TM_NORM_LAUNCH(1, true)
        }
        else {
            TM_NORM_LAUNCH(1, false)
        }
    }
#undef TM_NORM_LAUNCH
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}


// ---- fp32 residual stream -----------------------------------------------------------------------------------------------------------
// one workgroup per row: sum of squares in fp32 (per-thread partial sums in index order, then a fixed tree), two outputs from one statistic
template<class T>
__global__ __launch_bounds__(256) void rmsnorm_f32_kernel(T* __restrict__ y0, T* __restrict__ y1, int ldy, const float* __restrict__ x,
                                                          const int* __restrict__ rows, const float* __restrict__ w0,
                                                          const float* __restrict__ w1, float w_offset, float eps, int H)
{
    __shared__ float red[4];
    const int    m  = blockIdx.x;
    const float* xr = x + (size_t)(rows ? rows[m] : m) * H;
    float        ss = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        ss = fmaf(xr[i], xr[i], ss);
    }
    ss = group_sum<64>(ss);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = ss;
    }
    __syncthreads();
    const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += 256) {
        const float v = xr[i] * inv;
        y0[(size_t)m * ldy + i] = (T)(v * (w_offset + w0[i]));
        if (y1) {
            y1[(size_t)m * ldy + i] = (T)(v * (w_offset + w1[i]));
        }
    }
}

int launch_rmsnorm_f32(void* y0, void* y1, int ldy, int out_elem_bytes, const float* x, const int* rows, const float* w0, const float* w1,
                       float w_offset, float eps, int M, int H, hipStream_t st)
{
    TM_REQUIRE(y0 && x && w0 && (!y1 || w1) && ldy >= H && (out_elem_bytes == 2 || out_elem_bytes == 4), "rmsnorm_f32: operands");
    if (M == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        rmsnorm_f32_kernel<__bf16><<<M, 256, 0, st>>>((__bf16*)y0, (__bf16*)y1, ldy, x, rows, w0, w1, w_offset, eps, H);
    }
    else {
        rmsnorm_f32_kernel<float><<<M, 256, 0, st>>>((float*)y0, (float*)y1, ldy, x, rows, w0, w1, w_offset, eps, H);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// layer norm with bias, one workgroup per row; ADD: x[m] += LN(r[m]) and the new row is also written in the activation type
__device__ __forceinline__ float block_sum_256(float v, float* red)
{
    v = group_sum<64>(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = v;
    }
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
}

template<class T, bool ADD>
__global__ __launch_bounds__(256) void layernorm_f32_kernel(T* __restrict__ y, int ldy, float* __restrict__ xs, const float* __restrict__ src,
                                                            const int* __restrict__ rows, const float* __restrict__ w,
                                                            const float* __restrict__ b, float eps, int H)
{
    __shared__ float red[4];
    const int    m  = blockIdx.x;
    const float* r  = src + (size_t)(rows ? rows[m] : m) * H;
    float        sm = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        sm += r[i];
    }
    const float mean = block_sum_256(sm, red) / (float)H;
    float       ss   = 0.f;
    for (int i = threadIdx.x; i < H; i += 256) {
        const float d = r[i] - mean;
        ss            = fmaf(d, d, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)H + eps);
    for (int i = threadIdx.x; i < H; i += 256) {
        float v = fmaf((r[i] - mean) * inv, w[i], b[i]);
        if constexpr (ADD) {
            v += xs[(size_t)m * H + i];
            xs[(size_t)m * H + i] = v;
        }
        y[(size_t)m * ldy + i] = (T)v;
    }
}

// the same with the row held in registers (H <= 256 * NR): one pass over memory instead of three
template<class T, bool ADD, int NR>
__global__ __launch_bounds__(256) void layernorm_f32_reg_kernel(T* __restrict__ y, int ldy, float* __restrict__ xs, const float* __restrict__ src,
                                                                const int* __restrict__ rows, const float* __restrict__ w,
                                                                const float* __restrict__ b, float eps, int H)
{
    __shared__ float red[4];
    const int    m = blockIdx.x;
    const float* r = src + (size_t)(rows ? rows[m] : m) * H;
    float        v[NR], sm = 0.f;
#pragma unroll
    for (int q = 0; q < NR; ++q) {
        const int i = threadIdx.x + q * 256;
        v[q]        = i < H ? r[i] : 0.f;
        sm += v[q];
    }
    const float mean = block_sum_256(sm, red) / (float)H;
    float       ss   = 0.f;
#pragma unroll
    for (int q = 0; q < NR; ++q) {
        const float d = threadIdx.x + q * 256 < H ? v[q] - mean : 0.f;
        ss            = fmaf(d, d, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)H + eps);
#pragma unroll
    for (int q = 0; q < NR; ++q) {
        const int i = threadIdx.x + q * 256;
        if (i < H) {
            float o = fmaf((v[q] - mean) * inv, w[i], b[i]);
            if constexpr (ADD) {
                o += xs[(size_t)m * H + i];
                xs[(size_t)m * H + i] = o;
            }
            y[(size_t)m * ldy + i] = (T)o;
        }
    }
}

template<class T, bool ADD>
static void launch_layernorm_any(T* y, int ldy, float* xs, const float* src, const int* rows, const float* w, const float* b, float eps, int M, int H,
                                 hipStream_t st)
{
    if (H <= 1024) {
        layernorm_f32_reg_kernel<T, ADD, 4><<<M, 256, 0, st>>>(y, ldy, xs, src, rows, w, b, eps, H);
    }
    else if (H <= 4096) {
        layernorm_f32_reg_kernel<T, ADD, 16><<<M, 256, 0, st>>>(y, ldy, xs, src, rows, w, b, eps, H);
    }
    else if (H <= 8192) {
        layernorm_f32_reg_kernel<T, ADD, 32><<<M, 256, 0, st>>>(y, ldy, xs, src, rows, w, b, eps, H);
    }
    else {
        layernorm_f32_kernel<T, ADD><<<M, 256, 0, st>>>(y, ldy, xs, src, rows, w, b, eps, H);
    }
}

int launch_layernorm_f32(void* y, int ldy, int out_elem_bytes, const float* x, const int* rows, const float* w, const float* b, float eps, int M,
                         int H, hipStream_t st)
{
    TM_REQUIRE(y && x && w && b && ldy >= H && (out_elem_bytes == 2 || out_elem_bytes == 4), "layernorm_f32: operands");
    if (M == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        launch_layernorm_any<__bf16, false>((__bf16*)y, ldy, nullptr, x, rows, w, b, eps, M, H, st);
    }
    else {
        launch_layernorm_any<float, false>((float*)y, ldy, nullptr, x, rows, w, b, eps, M, H, st);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

int launch_layernorm_add_f32(float* x, void* h, int ldh, int h_elem_bytes, const float* r, const float* w, const float* b, float eps, int M, int H,
                             hipStream_t st)
{
    TM_REQUIRE(x && h && r && w && b && ldh >= H && (h_elem_bytes == 2 || h_elem_bytes == 4), "layernorm_add_f32: operands");
    if (M == 0) {
        return 0;
    }
    if (h_elem_bytes == 2) {
        launch_layernorm_any<__bf16, true>((__bf16*)h, ldh, x, r, nullptr, w, b, eps, M, H, st);
    }
    else {
        launch_layernorm_any<float, true>((float*)h, ldh, x, r, nullptr, w, b, eps, M, H, st);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// RMS norm in groups, one workgroup per row; the row is staged in LDS (H + groups floats), wave w reduces the groups w, w + 4, ...
// JOIN: the normed vector is 0.5 (r / rms(r) jw + r2 / rms(r2) jw2), each RMS over the whole row.  ADD: x[m] += GN(.), the new row is
// also written in the activation type
template<class T, bool ADD>
__global__ __launch_bounds__(256) void group_rmsnorm_f32_kernel(T* __restrict__ y, int ldy, float* __restrict__ xs, const float* __restrict__ src,
                                                                const float* __restrict__ src2, const float* __restrict__ jw,
                                                                const float* __restrict__ jw2, const int* __restrict__ rows,
                                                                const float* __restrict__ w, int groups, float eps, int H)
{
    extern __shared__ float gn_lds[];
    __shared__ float red[4];
    float*       row = gn_lds;
    float*       inv = gn_lds + H;
    const int    m = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const size_t r0 = (size_t)(rows ? rows[m] : m) * H;
    if (src2) {
        float s1 = 0.f, s2 = 0.f;
        for (int i = threadIdx.x; i < H; i += 256) {
            const float a = src[r0 + i], b = src2[r0 + i];
            s1 = fmaf(a, a, s1);
            s2 = fmaf(b, b, s2);
        }
        const float i1 = 1.0f / sqrtf(block_sum_256(s1, red) / (float)H + eps);
        const float i2 = 1.0f / sqrtf(block_sum_256(s2, red) / (float)H + eps);
        for (int i = threadIdx.x; i < H; i += 256) {
            row[i] = 0.5f * (src[r0 + i] * i1 * jw[i] + src2[r0 + i] * i2 * jw2[i]);
        }
    }
    else {
        for (int i = threadIdx.x; i < H; i += 256) {
            row[i] = src[r0 + i];
        }
    }
    __syncthreads();
    const int n = H / groups;
    for (int g = wave; g < groups; g += 4) {
        float ss = 0.f;
        for (int i = lane; i < n; i += 64) {
            const float v = row[g * n + i];
            ss            = fmaf(v, v, ss);
        }
        ss = group_sum<64>(ss);
        if (lane == 0) {
            inv[g] = 1.0f / sqrtf(ss / (float)n + eps);
        }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < H; i += 256) {
        float o = row[i] * inv[i / n] * w[i];
        if constexpr (ADD) {
            o += xs[(size_t)m * H + i];
            xs[(size_t)m * H + i] = o;
        }
        y[(size_t)m * ldy + i] = (T)o;
    }
}

int launch_group_rmsnorm_f32(void* y, int ldy, int out_elem_bytes, const float* x, const int* rows, const float* w, int groups, float eps, int M,
                             int H, hipStream_t st)
{
    TM_REQUIRE(y && x && w && ldy >= H && (out_elem_bytes == 2 || out_elem_bytes == 4), "group_rmsnorm_f32: operands");
    TM_REQUIRE(groups >= 1 && H % groups == 0 && H + groups <= 16000, "group_rmsnorm_f32: the width is a multiple of the groups, at most 16000 floats in LDS");
    if (M == 0) {
        return 0;
    }
    const size_t lds = (size_t)(H + groups) * 4;
    if (out_elem_bytes == 2) {
        group_rmsnorm_f32_kernel<__bf16, false><<<M, 256, lds, st>>>((__bf16*)y, ldy, nullptr, x, nullptr, nullptr, nullptr, rows, w, groups, eps, H);
    }
    else {
        group_rmsnorm_f32_kernel<float, false><<<M, 256, lds, st>>>((float*)y, ldy, nullptr, x, nullptr, nullptr, nullptr, rows, w, groups, eps, H);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

int launch_group_rmsnorm_add_f32(float* x, void* h, int ldh, int h_elem_bytes, const float* r, const float* r2, const float* jw, const float* jw2,
                                 const float* w, int groups, float eps, int M, int H, hipStream_t st)
{
    TM_REQUIRE(x && h && r && w && ldh >= H && (h_elem_bytes == 2 || h_elem_bytes == 4) && (!r2 || (jw && jw2)), "group_rmsnorm_add_f32: operands");
    TM_REQUIRE(groups >= 1 && H % groups == 0 && H + groups <= 16000, "group_rmsnorm_add_f32: the width is a multiple of the groups, at most 16000 floats in LDS");
    if (M == 0) {
        return 0;
    }
    const size_t lds = (size_t)(H + groups) * 4;
    if (h_elem_bytes == 2) {
        group_rmsnorm_f32_kernel<__bf16, true><<<M, 256, lds, st>>>((__bf16*)h, ldh, x, r, r2, jw, jw2, nullptr, w, groups, eps, H);
    }
    else {
        group_rmsnorm_f32_kernel<float, true><<<M, 256, lds, st>>>((float*)h, ldh, x, r, r2, jw, jw2, nullptr, w, groups, eps, H);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// y = act(x) in the activation type: the stream as a GEMM operand (act 0), tanh of a low-rank projection (act 1)
template<class T>
__global__ void act_cast_f32_kernel(T* __restrict__ y, int ldy, const float* __restrict__ x, int ldx, int M, int H, int act)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)M * H) {
        return;
    }
    const int   m = (int)(i / H), c = (int)(i % H);
    const float v = x[(size_t)m * ldx + c];
    y[(size_t)m * ldy + c] = (T)(act == 1 ? tanhf(v) : v);
}

int launch_act_cast_f32(void* y, int ldy, int out_elem_bytes, const float* x, int ldx, int M, int H, int act, hipStream_t st)
{
    TM_REQUIRE(y && x && ldy >= H && ldx >= H && (out_elem_bytes == 2 || out_elem_bytes == 4), "act_cast_f32: operands");
    const size_t total = (size_t)M * H;
    if (total == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        act_cast_f32_kernel<__bf16><<<(total + 255) / 256, 256, 0, st>>>((__bf16*)y, ldy, x, ldx, M, H, act);
    }
    else {
        act_cast_f32_kernel<float><<<(total + 255) / 256, 256, 0, st>>>((float*)y, ldy, x, ldx, M, H, act);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace tmk
