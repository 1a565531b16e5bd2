// Dense linears with unquantised weights: y = x . W^T for W stored [N][K] (the checkpoint's own orientation), in two number formats.
//
//   bf16 : weights and activations bfloat16, fp32 accumulation on the matrix cores (v_mfma_f32_16x16x32_bf16).  Both operands are
//          K-contiguous, so a lane's MFMA fragment (row = lane % 16, eight consecutive k at (lane / 16) * 8) is ONE 16-byte load.
//            * skinny kernel (M <= 32, the decode step): a wave owns 16 or 32 output columns, the four waves of a workgroup split K
//              and merge through LDS; weights stream straight from HBM into the fragments, one 256-wide chunk ahead of the MFMAs.
//            * tiled kernel (M > 32, prefill): 128 x 128 x 32 workgroup tiles staged in LDS (padded rows, no bank conflicts on the
//              16-byte fragment reads), 2 x 2 waves of 64 x 64, next tile prefetched into registers under the MFMAs.
//   fp32 : true 32-bit FMA arithmetic (no matrix-core shortcut, no reduced-precision mode), 64 x 64 x 16 LDS tiles, 4 x 4 per thread.
//
// Weights are kept as zero-padded images of Np x Kp elements (Np % 128 == 0, Kp % 32 == 0; bf16: in MFMA fragment order, see
// dense_frag_index; fp32: [Np][Kp]): no bounds test in any inner loop.  Activation rows
// have a leading dimension >= Kp; what lies in their pad columns only has to be finite, it meets zero weights.
//
// The epilogue is chosen per call (DenseEpilogue): plain store, relu(x)^2 (the squared-ReLU feed-forward), accumulate into the fp32
// residual stream with a multiplier (resid += alpha * acc: the output projection of a residual block closes the block in the GEMM),
// or alpha * acc as fp32 (scaled logits), acc + bias[n] as fp32, or the sigmoid-gated residual sum
// resid += sigmoid(gate[m][n] + gate_bias[n]) * acc (a block whose sublayers are gated element by element).
//
// A launch may be BATCHED (DenseCall::count > 1, grid z): item g multiplies with image g of the weight (images at a fixed stride), reads
// x at column g * x_col_stride and writes y at column g * y_col_stride -- per-head projections of one activation row -- or, with
// row_offsets, owns the rows [row_offsets[g], row_offsets[g + 1]) of x and y: the experts of a mixture over rows sorted by expert.
#include "tm_kernels.h"

namespace tmk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

template<class T>
__device__ __forceinline__ void dense_epilogue(void* y, int ldy, int m, int n, float acc, const DenseCall& c)
{
    const size_t i = (size_t)m * ldy + n;
    if (c.epi == kDenseStore) {
        ((T*)y)[i] = (T)acc;
    }
    else if (c.epi == kDenseRelu2) {
        const float r = fmaxf(acc, 0.f);
        ((T*)y)[i]    = (T)(r * r);
    }
    else if (c.epi == kDenseResidAdd) {
        ((float*)y)[i] += c.alpha * acc;
    }
    else if (c.epi == kDenseScaleF32) {
        ((float*)y)[i] = c.alpha * acc;
    }
    else if (c.epi == kDenseBiasF32) {
        ((float*)y)[i] = acc + c.bias[n];
    }
    else if (c.epi == kDenseXielu) {
        const float a = c.act_par[0], b = c.act_par[1];
        ((T*)y)[i]    = (T)(acc > 0.f ? fmaf(a * acc, acc, 0.5f * acc) : fmaf(b, expm1f(acc) - acc, 0.5f * acc));
    }
    else {  // kDenseResidGate
        const float z = c.gate[(size_t)m * c.ldg + n] + c.gate_bias[n];
        ((float*)y)[i] += acc / (1.f + expf(-z));
    }
}

// the item of a batched launch: where its operands start, and its row count (<= 0: nothing to do)
struct DenseItem {
    size_t x_off, w_off;
    int    row_base, col_base, M;
};
__device__ __forceinline__ DenseItem dense_item(const DenseCall& c, int g, int M, int ldx)
{
    DenseItem it{(size_t)g * c.x_col_stride, (size_t)g * c.w_stride, 0, g * c.y_col_stride, M};
    if (c.row_offsets) {
        it.row_base = c.row_offsets[g];
        it.x_off += (size_t)it.row_base * ldx;
        it.M = c.row_offsets[g + 1] - it.row_base;
    }
    return it;
}

// ---- bf16, M <= 32 ------------------------------------------------------------------------------------------------------------
// grid = ceil(N / (16 * NT)) workgroups of 4, 8 or 16 waves (narrow outputs with a long K: more waves split K so that the device still
// holds enough of them to cover the HBM latency).  A wave owns NT tiles of 16 output columns x MT tiles of 16 rows and every fourth
// k-chunk (eight 32-k MFMA steps with one column tile, four with two); an activation fragment serves the NT
// column tiles, a weight fragment the MT row tiles.  The weight stream is what comes from HBM, so it runs one chunk AHEAD in a second
// register buffer: the loads of chunk c + 1 are in flight under the activation reads (L2 hits) and MFMAs of chunk c.  The waves'
// partial sums meet in LDS.

template<int MT, int NT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void dense_skinny_bf16_kernel(const __bf16* __restrict__ x, int ldx, const __bf16* __restrict__ w, int Kp,
                                                                void* __restrict__ y, int ldy, int M, int N, DenseCall call)
{
    __shared__ float red[WAVES][MT * NT][64][4];
    const DenseItem it = dense_item(call, blockIdx.y, M, ldx);
    const int       row_base = it.row_base, col_base = it.col_base;
    M = it.M, x += it.x_off, w += it.w_off;
    if (M <= 0) {
        return;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0   = blockIdx.x * 16 * NT;
    const int r    = lane & 15, kc = (lane >> 4) * 8;
    const __bf16* wp[NT];
#pragma unroll
    for (int j = 0; j < NT; ++j) {
        // fragment order: block (tile, k / 32) at ((tile * Kp / 32 + k / 32) * 64 + lane) * 8 -- k advances by 16 elements per k.
        // Tiles up to Np / 16 exist (zero): no column test in the loop
        wp[j] = w + ((size_t)(n0 / 16 + j) * (Kp >> 5) * 64 + lane) * 8;
    }
    const __bf16* xp[MT];
    bool          xin[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xin[t] = t * 16 + r < M;
        xp[t]  = x + (size_t)(xin[t] ? t * 16 + r : 0) * ldx + kc;
    }
    floatx4 acc[MT][NT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
            acc[t][j] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
    // MFMA steps per chunk: two chunk buffers of KS x NT fragments must leave room for three to four waves per SIMD
    constexpr int kSkinnyKS = NT == 1 ? 8 : 4;
    const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8       wa[kSkinnyKS][NT], wb[kSkinnyKS][NT];
    auto fetch = [&](bf16x8 (&buf)[kSkinnyKS][NT], int k0) {
#pragma unroll
        for (int kk = 0; kk < kSkinnyKS; ++kk) {
            const int k = k0 + kk * 32;
#pragma unroll
            for (int j = 0; j < NT; ++j) {
                const bf16x8 v = *(const bf16x8*)(wp[j] + (size_t)min(k, Kp - 32) * 16);  // (k / 32) blocks of 512 elements; loads are
                buf[kk][j]     = k < Kp ? v : zero;                                        // unconditional so that all stay in flight
            }
        }
    };
    auto compute = [&](const bf16x8 (&buf)[kSkinnyKS][NT], int k0) {
#pragma unroll
        for (int kk = 0; kk < kSkinnyKS; ++kk) {
            const int k = k0 + kk * 32;
            if (k < Kp) {
                bf16x8 a[MT];
#pragma unroll
                for (int t = 0; t < MT; ++t) {
                    const bf16x8 v = *(const bf16x8*)(xp[t] + k);  // (rows beyond M read row 0)
                    a[t]           = xin[t] ? v : zero;
                }
#pragma unroll
                for (int t = 0; t < MT; ++t) {
#pragma unroll
                    for (int j = 0; j < NT; ++j) {
                        acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], buf[kk][j], acc[t][j], 0, 0, 0);
                    }
                }
            }
        }
    };
    constexpr int kChunk = kSkinnyKS * 32, kStride = WAVES * kChunk;  // the waves interleave their chunks
    int k0 = wave * kChunk;
    if (k0 < Kp) {
        fetch(wa, k0);
    }
    for (; k0 < Kp; k0 += 2 * kStride) {
        const int k1 = k0 + kStride, k2 = k1 + kStride;
        if (k1 < Kp) {
            fetch(wb, k1);
        }
        compute(wa, k0);
        if (k2 < Kp) {
            fetch(wa, k2);
        }
        if (k1 < Kp) {
            compute(wb, k1);
        }
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
#pragma unroll
        for (int j = 0; j < NT; ++j) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                red[wave][t * NT + j][lane][i] = acc[t][j][i];
            }
        }
    }
    __syncthreads();
    if (call.epi == kDenseGatedAct) {  // column tiles 2 j, 2 j + 1 of the image are the gate / up halves of output tile j
        if constexpr (NT == 2) {
            for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * 64) {
                const int t = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
                float     g = 0.f, u = 0.f;
#pragma unroll
                for (int wv = 0; wv < WAVES; wv += 4) {
                    g += (red[wv][t * 2][l][i] + red[wv + 1][t * 2][l][i]) + (red[wv + 2][t * 2][l][i] + red[wv + 3][t * 2][l][i]);
                    u += (red[wv][t * 2 + 1][l][i] + red[wv + 1][t * 2 + 1][l][i]) + (red[wv + 2][t * 2 + 1][l][i] + red[wv + 3][t * 2 + 1][l][i]);
                }
                const int m = t * 16 + (l >> 4) * 4 + i, n = (n0 >> 1) + (l & 15);
                if (m < M && n < call.n_out) {
                    ((__bf16*)y)[(size_t)(row_base + m) * ldy + col_base + n] = (__bf16)(act_apply(call.act, g) * u);
                }
            }
        }
        return;
    }
    for (int idx = threadIdx.x; idx < MT * NT * 256; idx += WAVES * 64) {
        const int tj = idx >> 8, l = (idx >> 2) & 63, i = idx & 3;
        float     s  = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; wv += 4) {  // fixed order: the result does not depend on which wave finished first
            s += (red[wv][tj][l][i] + red[wv + 1][tj][l][i]) + (red[wv + 2][tj][l][i] + red[wv + 3][tj][l][i]);
        }
        // C fragment: column = lane % 16, rows (lane / 16) * 4 + i
        const int m = (tj / NT) * 16 + (l >> 4) * 4 + i, n = n0 + (tj % NT) * 16 + (l & 15);
        if (m < M && n < N) {
            dense_epilogue<__bf16>(y, ldy, row_base + m, col_base + n, s, call);
        }
    }
}

// ---- bf16, tiled ----------------------------------------------------------------------------------------------------------------
constexpr int kTM = 128, kTN = 128, kTK = 32, kLdsRow = kTK + 8;  // 80-byte LDS rows: 16-byte fragment reads of 16 rows hit all banks once

__global__ __launch_bounds__(256) void dense_tiled_bf16_kernel(const __bf16* __restrict__ x, int ldx, const __bf16* __restrict__ w, int Kp,
                                                               void* __restrict__ y, int ldy, int M, int N, DenseCall call)
{
    __shared__ __attribute__((aligned(16))) __bf16 sa[2][kTM * kLdsRow];
    __shared__ __attribute__((aligned(16))) __bf16 sb[2][kTN * kLdsRow];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m0 = blockIdx.y * kTM, n0 = blockIdx.x * kTN;
    const DenseItem it = dense_item(call, blockIdx.z, M, ldx);
    const int       row_base = it.row_base, col_base = it.col_base;
    M = it.M, x += it.x_off, w += it.w_off;
    if (m0 >= M) {  // the whole workgroup: an item with fewer rows than the launch's largest
        return;
    }
    const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
    // staging: 128 rows x 32 k = 512 16-byte vectors per operand, two per thread: vector v -> row v / 4, k chunk (v % 4) * 8
    const int  sr0 = tid >> 2, sr1 = sr0 + 64, sk = (tid & 3) * 8;
    const bool a0 = m0 + sr0 < M, a1 = m0 + sr1 < M;
    const __bf16* ap0 = x + (size_t)(a0 ? m0 + sr0 : 0) * ldx + sk;
    const __bf16* ap1 = x + (size_t)(a1 ? m0 + sr1 : 0) * ldx + sk;
    // weights come in fragment order: vector v of a 128 x 32 tile = lane v % 64 of 16-row tile v / 64; it lands in the LDS row of that lane
    const int bt0 = tid >> 6, bt1 = bt0 + 4, bl = tid & 63;
    const int br0 = bt0 * 16 + (bl & 15), br1 = bt1 * 16 + (bl & 15), bk = (bl >> 4) * 8;
    const __bf16* bp0 = w + ((size_t)(n0 / 16 + bt0) * (Kp >> 5) * 64 + bl) * 8;
    const __bf16* bp1 = w + ((size_t)(n0 / 16 + bt1) * (Kp >> 5) * 64 + bl) * 8;
    const bf16x8  zero = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8        ra0, ra1, rb0, rb1;
    auto fetch = [&](int k) {
        const bf16x8 v0 = *(const bf16x8*)(ap0 + k), v1 = *(const bf16x8*)(ap1 + k);  // unconditional (rows beyond M read row 0)
        ra0 = a0 ? v0 : zero;
        ra1 = a1 ? v1 : zero;
        rb0 = *(const bf16x8*)(bp0 + (size_t)k * 16);
        rb1 = *(const bf16x8*)(bp1 + (size_t)k * 16);
    };
    auto stash = [&](int buf) {
        *(bf16x8*)(&sa[buf][sr0 * kLdsRow + sk]) = ra0;
        *(bf16x8*)(&sa[buf][sr1 * kLdsRow + sk]) = ra1;
        *(bf16x8*)(&sb[buf][br0 * kLdsRow + bk]) = rb0;
        *(bf16x8*)(&sb[buf][br1 * kLdsRow + bk]) = rb1;
    };
    floatx4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            acc[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
    const int fr = lane & 15, fk = (lane >> 4) * 8;
    fetch(0);
    stash(0);
    __syncthreads();
    const int steps = Kp / kTK;
    for (int s = 0; s < steps; ++s) {
        const int buf = s & 1;
        if (s + 1 < steps) {
            fetch((s + 1) * kTK);
        }
        bf16x8 fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            fa[i] = *(const bf16x8*)(&sa[buf][(wm + i * 16 + fr) * kLdsRow + fk]);
            fb[i] = *(const bf16x8*)(&sb[buf][(wn + i * 16 + fr) * kLdsRow + fk]);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
        if (s + 1 < steps) {
            stash(buf ^ 1);  // the other buffer: its readers finished before the barrier that ended step s - 1
        }
        __syncthreads();
    }
    if (call.epi == kDenseGatedAct) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 4; j += 2) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int m = m0 + wm + i * 16 + (lane >> 4) * 4 + q, n = ((n0 + wn) >> 1) + (j >> 1) * 16 + (lane & 15);
                    if (m < M && n < call.n_out) {
                        ((__bf16*)y)[(size_t)(row_base + m) * ldy + col_base + n] = (__bf16)(act_apply(call.act, acc[i][j][q]) * acc[i][j + 1][q]);
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int m = m0 + wm + i * 16 + (lane >> 4) * 4 + q, n = n0 + wn + j * 16 + (lane & 15);
                if (m < M && n < N) {
                    dense_epilogue<__bf16>(y, ldy, row_base + m, col_base + n, acc[i][j][q], call);
                }
            }
        }
    }
}

// ---- fp32 -------------------------------------------------------------------------------------------------------------------------
// 64 x 64 x 16 tiles, 256 threads, 4 x 4 outputs per thread; operands transposed into LDS ([k][row]) so that a thread's four rows /
// columns are one 16-byte read.  fmaf in k order: the result of a row does not depend on what shares its tile.
__global__ __launch_bounds__(256) void dense_f32_kernel(const float* __restrict__ x, int ldx, const float* __restrict__ w, int Kp,
                                                        void* __restrict__ y, int ldy, int M, int N, DenseCall call)
{
    __shared__ __attribute__((aligned(16))) float sa[16][64 + 4];
    __shared__ __attribute__((aligned(16))) float sb[16][64 + 4];
    const int tid = threadIdx.x;
    const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
    const DenseItem it = dense_item(call, blockIdx.z, M, ldx);
    const int       row_base = it.row_base, col_base = it.col_base;
    M = it.M, x += it.x_off, w += it.w_off;
    if (m0 >= M) {
        return;
    }
    const int tr = (tid >> 4) * 4, tc = (tid & 15) * 4;
    const int lr = tid >> 2, lk = (tid & 3) * 4;  // staging: row lr (0..63), k chunk lk (0, 4, 8, 12)
    const bool   ain = m0 + lr < M;
    const float* ap  = x + (size_t)(ain ? m0 + lr : 0) * ldx + lk;
    const float* bp  = w + (size_t)(n0 + lr) * Kp + lk;
    float        acc[4][4] = {};
    for (int k = 0; k < Kp; k += 16) {
        const floatx4 va = ain ? *(const floatx4*)(ap + k) : floatx4{0.f, 0.f, 0.f, 0.f};
        const floatx4 vb = *(const floatx4*)(bp + k);
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sa[lk + i][lr] = va[i];
            sb[lk + i][lr] = vb[i];
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            const floatx4 a = *(const floatx4*)(&sa[kk][tr]);
            const floatx4 b = *(const floatx4*)(&sb[kk][tc]);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
                }
            }
        }
    }
    if (call.epi == kDenseGatedAct) {  // a thread's columns are gate, gate, up, up of two outputs
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int m = m0 + tr + i, n = ((n0 + tc) >> 1) + j;
                if (m < M && n < call.n_out) {
                    ((float*)y)[(size_t)(row_base + m) * ldy + col_base + n] = act_apply(call.act, acc[i][j]) * acc[i][j + 2];
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int m = m0 + tr + i, n = n0 + tc + j;
            if (m < M && n < N) {
                dense_epilogue<float>(y, ldy, row_base + m, col_base + n, acc[i][j], call);
            }
        }
    }
}

// ---- weight images ----------------------------------------------------------------------------------------------------------------
// src: bf16 [rows][cols] (checkpoint bytes) -> dst[(row0 + r) * Kp + col0 + c], T = bf16 (copy) or float (exact widening)
// bf16 images are stored in FRAGMENT ORDER: the 16 rows x 32 k block (n / 16, k / 32) is one contiguous KB laid out as the 64 lanes of
// its MFMA fragment (lane = (k % 32) / 8 * 16 + n % 16, eight k each), blocks of one 16-row tile consecutive along k -- a wave's fragment
// load is one contiguous KB and a workgroup streams whole contiguous runs of HBM instead of 64-byte pieces of 16 rows
__host__ __device__ inline size_t dense_frag_index(int n, int k, int Kp)
{
    return ((((size_t)(n >> 4) * (Kp >> 5) + (k >> 5)) * 64 + ((k & 31) >> 3) * 16 + (n & 15)) << 3) + (k & 7);
}

template<class T>
__global__ void dense_place_kernel(T* __restrict__ dst, int Kp, int row0, int col0, const __bf16* __restrict__ src, int rows, int cols,
                                   int transpose, int half)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < (size_t)rows * cols) {
        const int r = (int)(i / cols), c = (int)(i % cols);
        int       n = row0 + (transpose ? c : r);  // transposed: the block's columns become output rows
        const int k = col0 + (transpose ? r : c);
        if (half) {
            n = dense_pair_row(n, half - 1, sizeof(T) == 4);
        }
        if constexpr (sizeof(T) == 2) {
            dst[dense_frag_index(n, k, Kp)] = (T)(float)src[i];
        }
        else {
            dst[(size_t)n * Kp + k] = (T)(float)src[i];
        }
    }
}

int dense_weight_alloc(DenseWeight& d, int K, int N, int dtype, hipStream_t st, int count)
{
    TM_REQUIRE(K >= 1 && N >= 1 && count >= 1 && (dtype == kDenseBf16 || dtype == kDenseF32), "dense weight: K, N, count >= 1, dtype bf16 | f32");
    d.K     = K;
    d.N     = N;
    d.Kp    = (K + 31) / 32 * 32;
    d.Np    = (N + 127) / 128 * 128;
    d.dtype = dtype;
    d.count = count;
    d.bytes = (size_t)d.Kp * d.Np * count * (dtype == kDenseF32 ? 4 : 2);
    TM_HIP_CHECK(hipMalloc(&d.w, d.bytes));
    TM_HIP_CHECK(hipMemsetAsync(d.w, 0, d.bytes, st));
    return 0;
}

int dense_weight_place(DenseWeight& d, int row0, int col0, const void* src_bf16, int rows, int cols, hipStream_t st, int item, bool transpose,
                       int half)
{
    TM_REQUIRE(d.w && row0 >= 0 && col0 >= 0 && item >= 0 && item < d.count && half >= 0 && half <= 2, "dense weight: part outside the image");
    TM_REQUIRE((half ? dense_pair_rows(row0 + (transpose ? cols : rows)) : row0 + (transpose ? cols : rows)) <= d.N
                   && col0 + (transpose ? rows : cols) <= d.K,
               "dense weight: part outside the image");
    const size_t n = (size_t)rows * cols, at = (size_t)item * d.Np * d.Kp;
    if (n == 0) {
        return 0;
    }
    if (d.dtype == kDenseF32) {
        dense_place_kernel<float><<<(n + 255) / 256, 256, 0, st>>>((float*)d.w + at, d.Kp, row0, col0, (const __bf16*)src_bf16, rows, cols, transpose, half);
    }
    else {
        dense_place_kernel<__bf16><<<(n + 255) / 256, 256, 0, st>>>((__bf16*)d.w + at, d.Kp, row0, col0, (const __bf16*)src_bf16, rows, cols, transpose, half);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

void dense_weight_free(DenseWeight& d)
{
    if (d.w) {
        (void)hipFree(d.w);
    }
    d.w = nullptr;
}

int launch_dense_linear(const DenseWeight& d, const void* x, int ldx, void* y, int ldy, int M, int epi, float alpha, hipStream_t st)
{
    DenseCall c;
    c.epi   = epi;
    c.alpha = alpha;
    return launch_dense_call(d, x, ldx, y, ldy, M, c, st);
}

int launch_dense_call(const DenseWeight& d, const void* x, int ldx, void* y, int ldy, int M, DenseCall call, hipStream_t st)
{
    const int epi = call.epi;
    TM_REQUIRE(d.w && x && y && M >= 0 && call.count >= 1 && call.count <= d.count, "dense linear: operands");
    const int n_y = epi == kDenseGatedAct ? call.n_out : d.N;
    TM_REQUIRE(ldx >= d.Kp + (call.count - 1) * call.x_col_stride && ldy >= n_y + (call.count - 1) * call.y_col_stride, "dense linear: row lengths");
    TM_REQUIRE(epi >= kDenseStore && epi <= kDenseXielu && (epi != kDenseXielu || call.act_par), "dense linear: epilogue");
    TM_REQUIRE(epi != kDenseGatedAct || (call.n_out >= 1 && dense_pair_rows(call.n_out) <= d.N), "dense linear: paired image");
    TM_REQUIRE(epi != kDenseBiasF32 || call.bias, "dense linear: bias");
    TM_REQUIRE(epi != kDenseResidGate || (call.gate && call.gate_bias && call.ldg >= d.N), "dense linear: gate");
    if (M == 0) {
        return 0;
    }
    call.w_stride = (size_t)d.Np * d.Kp;
    const int G   = call.count;
    if (d.dtype == kDenseF32) {
        TM_REQUIRE(ldx % 4 == 0, "dense linear (fp32): rows must be 16-byte aligned");
        TM_REQUIRE(call.x_col_stride % 4 == 0, "dense linear (fp32): items must be 16-byte aligned");
        dense_f32_kernel<<<dim3(d.Np / 64, (M + 63) / 64, G), 256, 0, st>>>((const float*)x, ldx, (const float*)d.w, d.Kp, y, ldy, M, d.N, call);
    }
    else {
        TM_REQUIRE(ldx % 8 == 0 && call.x_col_stride % 8 == 0, "dense linear (bf16): rows and items must be 16-byte aligned");
        if (M <= 32) {
            // two column tiles per wave where that still leaves >= 512 workgroups (two per CU): wide outputs amortise the activation reads
            const int nt     = (d.N >= 512 * 32 || epi == kDenseGatedAct) ? 2 : 1;  // (a gate / up pair is two adjacent tiles of one wave)
            const int wgs    = (d.N + 16 * nt - 1) / (16 * nt);
            const int chunk  = (nt == 1 ? 8 : 4) * 32;
            int       waves  = 4;  // ... and more waves per workgroup while the device holds fewer than 16 per CU and K has a chunk for each
            while (waves < (nt == 1 ? 16 : 8) && wgs * G * waves < 256 * 16 && d.Kp >= chunk * 2 * waves) {
                waves *= 2;
            }
#define TM_SKINNY(MT_, NT_, W_)                                                                                                     \
    dense_skinny_bf16_kernel<MT_, NT_, W_><<<dim3(wgs, G), W_ * 64, 0, st>>>((const __bf16*)x, ldx, (const __bf16*)d.w, d.Kp, y, ldy, M, d.N, call)
#define TM_SKINNY_W(MT_, NT_)                     \
    if (waves == 16 && NT_ == 1) {                \
        TM_SKINNY(MT_, 1, 16);                    \
    }                                             \
    else if (waves >= 8) {                        \
        TM_SKINNY(MT_, NT_, 8);                   \
    }                                             \
    else {                                        \
        TM_SKINNY(MT_, NT_, 4);                   \
    }
            if (M <= 16) {
                if (nt == 2) {
                    TM_SKINNY_W(1, 2)
                }
                else {
                    TM_SKINNY_W(1, 1)
                }
            }
            else {
                if (nt == 2) {
                    TM_SKINNY_W(2, 2)
                }
                else {
                    TM_SKINNY_W(2, 1)
                }
            }
#undef TM_SKINNY_W
#undef TM_SKINNY
        }
        else {
            dense_tiled_bf16_kernel<<<dim3(d.Np / kTN, (M + kTM - 1) / kTM, G), 256, 0, st>>>((const __bf16*)x, ldx, (const __bf16*)d.w, d.Kp, y,
                                                                                          ldy, M, d.N, call);
        }
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace tmk
