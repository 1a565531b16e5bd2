// Small HBM-bound helpers: embedding lookup, greedy argmax, row gather, unfused SiLU*up, and the
// group-wise u4 quantiser used to fabricate synthetic AWQ weights on the device.
//
// Replaces: embeddingLookup (src/turbomind/kernels/decoding_kernels.cu via language_model.cc:232),
//           top-k(=1) sampling (generation/sampling.cc:92-183), CollectHiddenStates
//           (unified_decoder.cc:355-372), Activation (kernels/activation.cu:27-130),
//           QuantizeGroupwise / IntegralQuantizer (kernels/quantization.cu:384-440,515-676).
#include "tm_common.h"
#include "tm_kernels.h"
#include <map>
#include <mutex>

namespace tmk {

__global__ __launch_bounds__(256) void embedding_kernel(half_t* __restrict__ out,
                                                        const half_t* __restrict__ table,
                                                        const int* __restrict__ ids,
                                                        int H,
                                                        int vocab)
{
    const int t  = blockIdx.x;
    int       id = ids[t];
    id           = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int v = threadIdx.x; v < H / 8; v += 256) {
        *(half8_t*)(out + (size_t)t * H + v * 8) = *(const half8_t*)(table + (size_t)id * H + v * 8);
    }
}

int launch_embedding(half_t* out, const half_t* table, const int* ids, int T, int H, int vocab, hipStream_t st)
{
    TM_REQUIRE(H % 8 == 0, "H % 8");
    if (T == 0) {
        return 0;
    }
    embedding_kernel<<<T, 256, 0, st>>>(out, table, ids, H, vocab);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

__global__ __launch_bounds__(256) void gather_rows_kernel(half_t* __restrict__ out,
                                                          const half_t* __restrict__ in,
                                                          const int* __restrict__ rows,
                                                          int H)
{
    const int r = rows[blockIdx.x];
    for (int v = threadIdx.x; v < H / 8; v += 256) {
        *(half8_t*)(out + (size_t)blockIdx.x * H + v * 8) = *(const half8_t*)(in + (size_t)r * H + v * 8);
    }
}

int launch_gather_rows(half_t* out, const half_t* in, const int* rows, int n, int H, hipStream_t st)
{
    if (n == 0) {
        return 0;
    }
    gather_rows_kernel<<<n, 256, 0, st>>>(out, in, rows, H);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// greedy: argmax over fp32-cast logits, lowest index wins ties. One 1024-thread workgroup per row.
__global__ __launch_bounds__(1024) void argmax_kernel(int* __restrict__ out_ids,
                                                      half_t* __restrict__ out_val,
                                                      const half_t* __restrict__ logits,
                                                      int V,
                                                      int ld,
                                                      int id_offset)
{
    __shared__ float sv[16];
    __shared__ int   si[16];
    const int     row  = blockIdx.x;
    const half_t* lp   = logits + (size_t)row * ld;
    float         best = -INFINITY;
    int           bi   = 0x7fffffff;
    const int     nvec = V / 8;
    for (int v = threadIdx.x; v < nvec; v += 1024) {
        const half8_t x = *(const half8_t*)(lp + (size_t)v * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float f = (float)x[e];
            if (f > best) {  // ascending scan: strict > keeps the lowest index
                best = f;
                bi   = v * 8 + e;
            }
        }
    }
    for (int i = nvec * 8 + threadIdx.x; i < V; i += 1024) {
        const float f = (float)lp[i];
        if (f > best || (f == best && i < bi)) {
            best = f;
            bi   = i;
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(best, off);
        const int   oi = __shfl_xor(bi, off);
        if (ov > best || (ov == best && oi < bi)) {
            best = ov;
            bi   = oi;
        }
    }
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) {
        sv[wave] = best;
        si[wave] = bi;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w) {
            if (sv[w] > best || (sv[w] == best && si[w] < bi)) {
                best = sv[w];
                bi   = si[w];
            }
        }
        out_ids[row] = (bi == 0x7fffffff ? 0 : bi) + id_offset;
        if (out_val) {
            out_val[row] = (half_t)best;
        }
    }
}

int launch_argmax(int* out_ids, half_t* out_val, const half_t* logits, int B, int V, int ld, int id_offset, hipStream_t st)
{
    TM_REQUIRE(ld % 8 == 0, "logits rows must be 16-byte aligned");
    if (B == 0) {
        return 0;
    }
    argmax_kernel<<<B, 1024, 0, st>>>(out_ids, out_val, logits, V, ld, id_offset);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// unfused activation on a [M][2*inter] buffer laid out [gate | up]
// Pseudo-random fp16 values in (-amp, amp) -- stand-in activations for the start-up GEMM tuner.  Not zeros: the matrix pipe
// of MI355X is power-limited, and a GEMM over all-zero activations runs at the full 2.4 GHz instead of the ~1.6 GHz it sustains
// on real data (measured: the fused w1w3 prefill tile 1152 us on zeros, 1697 us on N(0,1) rows) -- timings on zeros rank
// compute-bound candidates wrongly.
__global__ __launch_bounds__(256) void fill_uniform_f16_kernel(half_t* __restrict__ out, size_t n, float amp, uint32_t seed)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    uint32_t h = (uint32_t)i * 0x9E3779B1u + (uint32_t)(i >> 32) + seed;  // one round of a 32-bit integer hash
    h ^= h >> 16;
    h *= 0x7feb352du;
    h ^= h >> 15;
    h *= 0x846ca68bu;
    h ^= h >> 16;
    out[i] = (half_t)(((float)(h >> 8) * (1.0f / 8388608.0f) - 1.0f) * amp);
}

int launch_fill_uniform_f16(half_t* out, size_t n, float amp, uint32_t seed, hipStream_t st)
{
    if (n == 0) {
        return 0;
    }
    fill_uniform_f16_kernel<<<(unsigned)((n + 255) / 256), 256, 0, st>>>(out, n, amp, seed);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

__global__ __launch_bounds__(256) void silu_mul_kernel(half_t* __restrict__ out,
                                                       const half_t* __restrict__ gate_up,
                                                       int M,
                                                       int inter)
{
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (size_t)M * inter / 8) {
        return;
    }
    const int     m = idx / (inter / 8);
    const int     c = (idx - (size_t)m * (inter / 8)) * 8;
    const half8_t g = *(const half8_t*)(gate_up + (size_t)m * 2 * inter + c);
    const half8_t u = *(const half8_t*)(gate_up + (size_t)m * 2 * inter + inter + c);
    half8_t       o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const float gf = (float)g[e];
        o[e]           = (half_t)((gf / (1.0f + __builtin_expf(-gf))) * (float)u[e]);
    }
    *(half8_t*)(out + (size_t)m * inter + c) = o;
}

int launch_silu_mul(half_t* out, const half_t* gate_up, int M, int inter, hipStream_t st)
{
    TM_REQUIRE(inter % 8 == 0, "inter % 8");
    const size_t total = (size_t)M * inter / 8;
    if (total == 0) {
        return 0;
    }
    silu_mul_kernel<<<(total + 255) / 256, 256, 0, st>>>(out, gate_up, M, inter);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// IntegralQuantizer<half,4>: groups of `group` along K for every output column n.
//   scale_ = max(max-min, 1e-5)/15 ; zero_ = clamp(-rint(min/scale_), 0, 15)
//   q = clamp(rint(x/scale_) + zero_, 0, 15) ; d = h(q - zero_) * h(scale_)
// Output in the boundary layout: qweight int32 [K][N/8] (nibble j of word c = column 8c+j).
__global__ __launch_bounds__(256) void quantize_groupwise_u4_kernel(int32_t* __restrict__ qweight,
                                                                    half_t* __restrict__ scales,
                                                                    half_t* __restrict__ zeros,
                                                                    half_t* __restrict__ dequant,
                                                                    const half_t* __restrict__ w,
                                                                    int K,
                                                                    int N,
                                                                    int group)
{
    // one thread per (group, 8 consecutive columns)
    const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int    nc  = N / 8;
    if (idx >= (size_t)(K / group) * nc) {
        return;
    }
    const int gi = idx / nc;
    const int c  = idx - (size_t)gi * nc;
    float     mn[8], mx[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        mn[e] = INFINITY;
        mx[e] = -INFINITY;
    }
    for (int k = gi * group; k < (gi + 1) * group; ++k) {
        const half8_t x = *(const half8_t*)(w + (size_t)k * N + c * 8);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            mn[e] = fminf(mn[e], (float)x[e]);
            mx[e] = fmaxf(mx[e], (float)x[e]);
        }
    }
    float sc[8];
    int   zp[8];
    half8_t s_out, z_out;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        sc[e]    = fmaxf(mx[e] - mn[e], 1e-5f) / 15.0f;
        int z    = (int)(-__builtin_rintf(mn[e] / sc[e]));
        zp[e]    = z < 0 ? 0 : (z > 15 ? 15 : z);
        s_out[e] = (half_t)sc[e];
        z_out[e] = (half_t)(float)zp[e];
    }
    *(half8_t*)(scales + (size_t)gi * N + c * 8) = s_out;
    *(half8_t*)(zeros + (size_t)gi * N + c * 8)  = z_out;
    for (int k = gi * group; k < (gi + 1) * group; ++k) {
        const half8_t x = *(const half8_t*)(w + (size_t)k * N + c * 8);
        uint32_t      word = 0;
        half8_t       d;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            int q = (int)__builtin_rintf((float)x[e] / sc[e]) + zp[e];
            q     = q < 0 ? 0 : (q > 15 ? 15 : q);
            word |= (uint32_t)q << (4 * e);
            d[e] = (half_t)(float)(q - zp[e]) * s_out[e];
        }
        qweight[(size_t)k * nc + c] = (int32_t)word;
        if (dequant) {
            *(half8_t*)(dequant + (size_t)k * N + c * 8) = d;
        }
    }
}

int launch_quantize_groupwise_u4(int32_t* qweight, half_t* scales, half_t* zeros, half_t* dequant, const half_t* w,
                                 int K, int N, int group, hipStream_t st)
{
    TM_REQUIRE(N % 8 == 0 && K % group == 0, "N % 8 == 0, K % group == 0");
    const size_t total = (size_t)(K / group) * (N / 8);
    if (total == 0) {
        return 0;
    }
    quantize_groupwise_u4_kernel<<<(total + 255) / 256, 256, 0, st>>>(qweight, scales, zeros, dequant, w, K, N, group);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

int ensure_dynamic_lds(const void* kernel, int bytes)
{
    static std::mutex                               mu;
    static std::map<std::pair<const void*, int>, int> done;  // (kernel, device) -> bytes granted
    int dev = 0;
    TM_HIP_CHECK(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(mu);
    auto                        it = done.find({kernel, dev});
    if (it != done.end() && it->second >= bytes) {
        return 0;
    }
    TM_HIP_CHECK(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
    done[{kernel, dev}] = bytes;
    return 0;
}


template<class T>
__global__ void embedding_f32_kernel(float* __restrict__ out, const T* __restrict__ table, const int* __restrict__ ids, int T_, int H, int vocab,
                                     float scale)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (size_t)T_ * H) {
        const int t = (int)(i / H), c = (int)(i % H);
        int       id = ids[t];
        id           = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
        out[i]       = (float)table[(size_t)id * H + c] * scale;
    }
}

int launch_embedding_f32(float* out, const void* table, int table_elem_bytes, const int* ids, int T, int H, int vocab, hipStream_t st, float scale)
{
    TM_REQUIRE(out && table && ids && (table_elem_bytes == 2 || table_elem_bytes == 4), "embedding_f32: operands");
    const size_t n = (size_t)T * H;
    if (n == 0) {
        return 0;
    }
    if (table_elem_bytes == 2) {
        embedding_f32_kernel<__bf16><<<(n + 255) / 256, 256, 0, st>>>(out, (const __bf16*)table, ids, T, H, vocab, scale);
    }
    else {
        embedding_f32_kernel<float><<<(n + 255) / 256, 256, 0, st>>>(out, (const float*)table, ids, T, H, vocab, scale);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

__global__ void f32_to_f16_rows_kernel(half_t* __restrict__ out, int ld, const float* __restrict__ in, int n, int V)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (size_t)n * ld) {
        const int r = (int)(i / ld), c = (int)(i % ld);
        const float v = c < V ? in[(size_t)r * V + c] : -65504.f;  // pad columns can never win an arg-max
        out[i] = (half_t)fminf(fmaxf(v, -65504.f), 65504.f);
    }
}

int launch_f32_to_f16_rows(half_t* out, int ld, const float* in, int n, int V, hipStream_t st)
{
    TM_REQUIRE(out && in && ld >= V, "f32_to_f16_rows: operands");
    const size_t cnt = (size_t)n * ld;
    if (cnt > 0) {
        f32_to_f16_rows_kernel<<<(cnt + 255) / 256, 256, 0, st>>>(out, ld, in, n, V);
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}

// ---- fp32 stream helpers of the layer-list family ------------------------------------------------------------------------------------
// out[m] = [a[m] | b[m]] in the activation type: two fp32 streams side by side as the operand of one product
template<class T>
__global__ void concat2_kernel(T* __restrict__ out, int ldo, const float* __restrict__ a, const float* __restrict__ b, int H, size_t total)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < total) {
        const size_t m = i / (2 * H);
        const int    c = (int)(i % (2 * H));
        out[m * ldo + c] = (T)(c < H ? a[m * H + c] : b[m * H + c - H]);
    }
}

int launch_concat2(void* out, int ldo, int out_elem_bytes, const float* a, const float* b, int M, int H, hipStream_t st)
{
    TM_REQUIRE(out && a && b && ldo >= 2 * H && (out_elem_bytes == 2 || out_elem_bytes == 4), "concat2: operands");
    const size_t total = (size_t)M * 2 * H;
    if (total == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        concat2_kernel<__bf16><<<(total + 255) / 256, 256, 0, st>>>((__bf16*)out, ldo, a, b, H, total);
    }
    else {
        concat2_kernel<float><<<(total + 255) / 256, 256, 0, st>>>((float*)out, ldo, a, b, H, total);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// ---- mixer outputs on their way to the output projection ------------------------------------------------------------------------------
// differential attention: one wave per (row, head) joins the head's two maps, o = a1 - lambda a2, and scales o to unit RMS (times mult)
template<class T>
__global__ __launch_bounds__(256) void diff_head_norm_kernel(T* __restrict__ y, int ldy, const float* __restrict__ a, int lda,
                                                             const float* __restrict__ lambda, float mult, int heads, int n, float eps)
{
    const int t = blockIdx.x, h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= heads) {
        return;
    }
    const float  lam = lambda[0];
    const float *a1 = a + (size_t)t * lda + (size_t)h * n, *a2 = a1 + (size_t)heads * n;
    float        ss = 0.f;
    for (int i = lane; i < n; i += 64) {
        const float o = fmaf(-lam, a2[i], a1[i]);
        ss            = fmaf(o, o, ss);
    }
    const float inv = mult / sqrtf(group_sum<64>(ss) / (float)n + eps);
    for (int i = lane; i < n; i += 64) {
        y[(size_t)t * ldy + (size_t)h * n + i] = (T)(fmaf(-lam, a2[i], a1[i]) * inv);
    }
}

int launch_diff_head_norm(void* y, int ldy, int out_elem_bytes, const float* a, int lda, const float* lambda, float mult, int rows, int heads, int n,
                          float eps, hipStream_t st)
{
    TM_REQUIRE(y && a && lambda && heads >= 1 && n >= 1 && ldy >= heads * n && lda >= 2 * heads * n && (out_elem_bytes == 2 || out_elem_bytes == 4),
               "diff_head_norm: operands");
    if (rows == 0) {
        return 0;
    }
    const dim3 grid(rows, (heads + 3) / 4);
    if (out_elem_bytes == 2) {
        diff_head_norm_kernel<__bf16><<<grid, 256, 0, st>>>((__bf16*)y, ldy, a, lda, lambda, mult, heads, n, eps);
    }
    else {
        diff_head_norm_kernel<float><<<grid, 256, 0, st>>>((float*)y, ldy, a, lda, lambda, mult, heads, n, eps);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

template<class T>
__global__ void sigmoid_gate_mul_kernel(T* __restrict__ y, int ldy, const float* __restrict__ x, int ldx, const float* __restrict__ gate, int ldg,
                                        int rows, int n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (size_t)rows * n) {
        const int t = (int)(i / n), c = (int)(i % n);
        y[(size_t)t * ldy + c] = (T)(x[(size_t)t * ldx + c] / (1.f + expf(-gate[(size_t)t * ldg + c])));
    }
}

int launch_sigmoid_gate_mul(void* y, int ldy, int out_elem_bytes, const float* x, int ldx, const float* gate, int ldg, int rows, int n, hipStream_t st)
{
    TM_REQUIRE(y && x && gate && n >= 1 && ldy >= n && ldx >= n && ldg >= n && (out_elem_bytes == 2 || out_elem_bytes == 4), "sigmoid_gate_mul: operands");
    const size_t total = (size_t)rows * n;
    if (total == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        sigmoid_gate_mul_kernel<__bf16><<<(total + 255) / 256, 256, 0, st>>>((__bf16*)y, ldy, x, ldx, gate, ldg, rows, n);
    }
    else {
        sigmoid_gate_mul_kernel<float><<<(total + 255) / 256, 256, 0, st>>>((float*)y, ldy, x, ldx, gate, ldg, rows, n);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

__global__ void softcap_f32_kernel(float* __restrict__ x, size_t n, float cap)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        x[i] = cap * tanhf(x[i] / cap);
    }
}

int launch_softcap_f32(float* x, size_t n, float cap, hipStream_t st)
{
    TM_REQUIRE(x && cap > 0.f, "softcap_f32: operands");
    if (n > 0) {
        softcap_f32_kernel<<<(n + 255) / 256, 256, 0, st>>>(x, n, cap);
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}

}  // namespace tmk
