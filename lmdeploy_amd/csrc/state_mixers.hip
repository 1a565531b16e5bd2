// Mixers with a recurrent state instead of a key / value cache: per head a matrix S [dim][vdim] in fp32 that every token updates.
//
//   linear attention ("lightning"):  S <- decay[head] S + k v^T                         o = S^T q      q, k, v = silu(projection)
//   generalized delta rule:          S <- diag(w) S - (a u)(u^T S) + k v^T              o = S^T r      u = k / sqrt(|k|^2 + 1e-6),
//                                    w, a per key channel (both terms read the old S)
//   gated delta rule:                S <- diag(g) S;  S <- S + k (beta (v - S^T k))^T   o = S^T q      is the same recurrence with
//                                    w = g, u = g k, a u = beta k and the key beta k (launch_gdelta_prep forms these vectors)
//   short convolution:               y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel; its state is the last taps - 1 inputs
//
// State pool: one state per (slot, layer run) -- slot = the engine's batch slot of the sequence, plus one parking slot for the decode
// rows of slots that hold no running sequence.  A sequence whose first row of a launch has position 0 starts from zero whatever the
// slot holds (slots are reused without clearing).  Everything here is fp32 in both number formats of the engine.
//
// The columns of S evolve independently (S[:, j] only meets v[j]), so the work is split over (sequence, head, 16 value columns): one wave
// owns a [dim][16] slab -- lane = (column pair c = lane % 8, row group rg = lane / 8), rows rg * dq + ii, dq = ceil(dim / 8), columns
// 2 c and 2 c + 1: DQ x 2 registers -- and walks the sequence's rows of this launch in order; the reductions over the key channels are a
// register sum + three lane shuffles.  (Two columns per lane: every per-token vector element read from LDS feeds two multiply-adds;
// with one the kernel is bound by LDS reads.)  Four waves (64 value columns) share a workgroup and the LDS stage of the per-token
// vectors (q, k, and w, a u, u for the delta rule), loaded TB tokens at a time: the next stage's global loads are issued before the
// current stage's tokens are walked and land in the other LDS buffer afterwards, so their latency hides under the recurrence.  A slab is
// stored as the wave holds it, [ii][column of the pair][lane]: loading and storing it are fully coalesced.
// The delta rule walks its tokens one by one (two dependent reductions per token).  Linear attention with its scalar decay takes a whole
// stage of T <= TB tokens at once, which replaces T dependent steps by independent sums:
//   o_t = decay^(t+1) S0^T q_t + sum_{j <= t} decay^(t-j) (q_t . k_j) v_j          S_T = decay^T S0 + sum_j decay^(T-1-j) k_j v_j^T
// -- the pair products (q_t . k_j) decay^(t-j) are formed once per workgroup (one thread per pair) and shared by all columns.
// One kernel serves prompt portions (many rows per sequence) and decoded tokens (one row, TB = 1): the state traffic of a decode step,
// 2 * dim * vdim * 4 bytes per head, is what bounds it.
#include "tm_kernels.h"

namespace tmk {

constexpr int kStateCW = 8;   // lanes per row group; 64 / kStateCW row groups
constexpr int kStateNC = 2;   // value columns per lane: a wave owns kStateCW * kStateNC columns

__device__ __forceinline__ float sm_silu(float z)
{
    return z / (1.f + expf(-z));
}

size_t state_mix_floats(int heads, int dim, int vdim)
{
    const int wcols = kStateCW * kStateNC;
    return (size_t)heads * ((vdim + wcols - 1) / wcols) * ((dim + 7) / 8) * 64 * kStateNC;
}

// grid (nseq, heads, ceil(vdim / 64)), 256 threads, dynamic LDS = 2 * tb * (NV * dim + 64) floats (+ TB * TB for linear attention); NV = 2 | 5
// staged vectors per token, tb = min(TB, max_q_len) tokens per stage, TB: as many as keep the buffers under 64 KB.
// EXACT: dim == 8 * DQ -- every LDS stride is a compile-time constant and the per-token vectors are read 16 bytes at a time
template<int DQ, bool DELTA, int TB, bool EXACT>
__global__ __launch_bounds__(256) void state_mix_kernel(StateMixParams p)
{
    extern __shared__ __attribute__((aligned(16))) float lds_all[];
    constexpr int NV = DELTA ? 5 : 2, CW = kStateCW, NC = kStateNC, RG = 64 / CW, WV = CW * NC, WC = 4 * WV;
    constexpr int PER  = (TB * DQ * RG + 255) / 256;  // staged elements per vector and thread (dim <= DQ * RG)
    constexpr int VPER = (TB * WC + 255) / 256;
    static_assert(TB * TB <= 256, "one thread per token pair");
    const int s = blockIdx.x, h = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int D = EXACT ? DQ * RG : p.dim, V = p.vdim, dq = EXACT ? DQ : (D + RG - 1) / RG, ncb = (V + WV - 1) / WV;
    const int Dp = dq * RG;  // staged vectors are padded to the row groups' share (zeros behind dim)
    const int cb = blockIdx.z * 4 + wave, c = lane % CW, rg = lane / CW, j0 = cb * WV + c * NC;
    const bool wave_on = cb < ncb;
    const int row0 = p.cu_q[s] - p.cu_q[0], q_len = p.cu_q[s + 1] - p.cu_q[s];
    const int pos0 = p.k_len[s] - q_len;
    int       slot = p.seq_slot ? p.seq_slot[s] : p.slot0 + s;
    if (p.active && !p.active[s]) {
        slot = p.park_slot;
    }
    float* slab = p.state + (size_t)slot * p.slot_stride + p.layer_offset + ((size_t)h * ncb + (wave_on ? cb : 0)) * dq * 64 * NC;
    float  S[DQ][NC];
#pragma unroll
    for (int ii = 0; ii < DQ; ++ii) {
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            S[ii][n] = (wave_on && pos0 > 0 && ii < dq) ? slab[(ii * NC + n) * 64 + lane] : 0.f;
        }
    }
    const float  decay = DELTA ? 0.f : p.decay_h[h];
    const int    tb    = min(TB, p.max_q_len);
    const size_t stage = (size_t)tb * (NV * Dp + WC);  // floats of one LDS buffer: [tb][NV][Dp] vectors, then [tb][WC] values
    float        rv[NV][PER], rval[VPER];
    // global loads of the stage that starts at token t0 (into registers) / their way into LDS buffer `buf`
    auto fetch = [&](int t0) {
        const int nt = min(tb, q_len - t0);
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int  i  = threadIdx.x + r * 256;
            const bool ok = i < nt * Dp && i % Dp < D;
            const int  t = ok ? i / Dp : 0, d = ok ? i % Dp : 0;
            const size_t row = (size_t)(row0 + t0 + t);
            const float* pr  = p.proj + row * p.ld + h * D + d;
            rv[0][r] = ok ? pr[p.c_q] : 0.f;
            rv[1][r] = ok ? pr[p.c_k] : 0.f;
            if constexpr (DELTA) {
                rv[2][r] = ok ? p.decay_w[row * p.ld_w + h * D + d] : 0.f;
                rv[3][r] = ok ? pr[p.c_a] : 0.f;
                rv[4][r] = ok ? p.unit[row * p.ld_u + h * D + d] : 0.f;
            }
        }
#pragma unroll
        for (int r = 0; r < VPER; ++r) {
            const int i = threadIdx.x + r * 256;
            const int t = i / WC, jj = blockIdx.z * WC + i % WC;
            rval[r]     = (i < nt * WC && jj < V) ? p.proj[(size_t)(row0 + t0 + t) * p.ld + p.c_v + h * V + jj] : 0.f;
        }
    };
    auto park = [&](int t0, int buf) {
        const int nt  = min(tb, q_len - t0);
        float*    lds = lds_all + buf * stage;
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int i = threadIdx.x + r * 256;
            if (i < nt * Dp) {
                const int t = i / Dp, d = i % Dp;
#pragma unroll
                for (int v = 0; v < NV; ++v) {
                    lds[(t * NV + v) * Dp + d] = DELTA ? rv[v][r] : sm_silu(rv[v][r]);
                }
            }
        }
#pragma unroll
        for (int r = 0; r < VPER; ++r) {
            const int i = threadIdx.x + r * 256;
            if (i < nt * WC) {
                lds[(size_t)tb * NV * Dp + i] = DELTA ? rval[r] : sm_silu(rval[r]);
            }
        }
    };
    // linear attention: powers of the decay, and this thread's pair (t, j) of the stage's token-by-token products
    float     pwr[TB + 1], pair_pow = 1.f;
    const int pt = threadIdx.x / TB, pj = threadIdx.x % TB;
    float*    Pm = lds_all + 2 * stage;  // [TB][TB] (q_t . k_j) decay^(t - j), zero where j > t or t is not in the stage
    if constexpr (!DELTA) {
        pwr[0] = 1.f;
#pragma unroll
        for (int n = 1; n <= TB; ++n) {
            pwr[n] = pwr[n - 1] * decay;
        }
        for (int n = 0; pt < TB && n < pt - pj; ++n) {
            pair_pow *= decay;
        }
    }
    auto reduce_rg = [&](float a) {
        a += __shfl_xor(a, 8);
        a += __shfl_xor(a, 16);
        return a + __shfl_xor(a, 32);
    };
    auto store_out = [&](int t, const float (&o)[NC]) {
        float* out = p.out + (size_t)(row0 + t) * p.ldo + h * V + j0;
#pragma unroll
        for (int n = 0; n < NC; ++n) {
            if (j0 + n < V) {
                out[n] = o[n];
            }
        }
    };
    fetch(0);
    park(0, 0);
    __syncthreads();
    int buf = 0;
    for (int t0 = 0; t0 < q_len; t0 += tb, buf ^= 1) {
        const int  nt   = min(tb, q_len - t0);
        const bool more = t0 + tb < q_len;
        if (more) {
            fetch(t0 + tb);
        }
        const float* lds = lds_all + buf * stage;
        const float* sv  = lds + (size_t)tb * NV * Dp + wave * WV + c * NC;  // the lane's columns of token t at sv[t * WC + n]
        if constexpr (!DELTA) {
            if (threadIdx.x < TB * TB) {
                float dot = 0.f;
                if (pt < nt && pj <= pt) {
                    const float* qt = lds + (size_t)(pt * NV + 0) * Dp;
                    const float* kj = lds + (size_t)(pj * NV + 1) * Dp;
                    // (every thread starts at another channel: the threads of a wave read different LDS banks)
                    if constexpr (EXACT) {
                        for (int d4 = 0; d4 < Dp / 4; ++d4) {
                            const int     i = ((d4 + pj) % (Dp / 4)) * 4;
                            const floatx4 a = *(const floatx4*)(qt + i), b = *(const floatx4*)(kj + i);
                            dot = fmaf(a[0], b[0], fmaf(a[1], b[1], fmaf(a[2], b[2], fmaf(a[3], b[3], dot))));
                        }
                    }
                    else {
                        for (int d = 0; d < Dp; ++d) {
                            const int i = (d + pj) % Dp;
                            dot         = fmaf(qt[i], kj[i], dot);
                        }
                    }
                    dot *= pair_pow;
                }
                Pm[pt * TB + pj] = dot;
            }
            __syncthreads();
            if (wave_on) {
                float acc[TB][NC];
#pragma unroll
                for (int t = 0; t < TB; ++t) {  // what the old state answers to every query of the stage
#pragma unroll
                    for (int n = 0; n < NC; ++n) {
                        acc[t][n] = 0.f;
                    }
                    if (t < nt) {
                        const float* q = lds + (size_t)(t * NV + 0) * Dp + rg * dq;
#pragma unroll
                        for (int ii = 0; ii < DQ; ++ii) {
                            if (EXACT || ii < dq) {
                                const float qv = q[ii];
#pragma unroll
                                for (int n = 0; n < NC; ++n) {
                                    acc[t][n] = fmaf(S[ii][n], qv, acc[t][n]);
                                }
                            }
                        }
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            acc[t][n] *= pwr[t + 1];
                        }
                    }
                }
#pragma unroll
                for (int m = 0; m < (TB + RG - 1) / RG; ++m) {  // the stage's own tokens: row group rg adds tokens rg, rg + 8, ...
                    const int jt = rg + RG * m;
                    if (jt < TB) {
                        float vj[NC];
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            vj[n] = jt < nt ? sv[jt * WC + n] : 0.f;
                        }
#pragma unroll
                        for (int t = 0; t < TB; ++t) {
                            const float pw = Pm[t * TB + jt];
#pragma unroll
                            for (int n = 0; n < NC; ++n) {
                                acc[t][n] = fmaf(pw, vj[n], acc[t][n]);
                            }
                        }
                    }
                }
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    if (t < nt) {
                        float o[NC];
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            o[n] = reduce_rg(acc[t][n]);
                        }
                        if ((t & (RG - 1)) == rg) {
                            store_out(t0 + t, o);
                        }
                    }
                }
                float dn = 1.f;
#pragma unroll
                for (int t = 0; t < TB; ++t) {
                    dn *= t < nt ? decay : 1.f;
                }
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
#pragma unroll
                    for (int n = 0; n < NC; ++n) {
                        S[ii][n] *= dn;
                    }
                }
                float wgt = 1.f;  // decay^(nt - 1 - token)
#pragma unroll
                for (int t = TB - 1; t >= 0; --t) {
                    if (t < nt) {
                        const float* k = lds + (size_t)(t * NV + 1) * Dp + rg * dq;
                        float        wv[NC];
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            wv[n] = wgt * sv[t * WC + n];
                        }
#pragma unroll
                        for (int ii = 0; ii < DQ; ++ii) {
                            if (EXACT || ii < dq) {
                                const float kv = k[ii];
#pragma unroll
                                for (int n = 0; n < NC; ++n) {
                                    S[ii][n] = fmaf(kv, wv[n], S[ii][n]);
                                }
                            }
                        }
                        wgt *= decay;
                    }
                }
            }
        }
        else {
            for (int t = 0; wave_on && t < nt; ++t) {
                const float* q  = lds + (size_t)(t * NV + 0) * Dp + rg * dq;
                const float* k  = lds + (size_t)(t * NV + 1) * Dp + rg * dq;
                const float* w  = lds + (size_t)(t * NV + 2) * Dp + rg * dq;
                const float* au = lds + (size_t)(t * NV + 3) * Dp + rg * dq;
                const float* u  = lds + (size_t)(t * NV + 4) * Dp + rg * dq;
                float        v[NC], us[NC], acc[NC];
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    v[n]  = sv[t * WC + n];
                    us[n] = acc[n] = 0.f;
                }
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
                    if (EXACT || ii < dq) {  // (rows behind dim meet staged zeros and stay zero)
                        const float uv = u[ii];
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            us[n] = fmaf(uv, S[ii][n], us[n]);
                        }
                    }
                }
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    us[n] = reduce_rg(us[n]);
                }
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
                    if (EXACT || ii < dq) {
                        const float wv = w[ii], av = au[ii], kv = k[ii], qv = q[ii];
#pragma unroll
                        for (int n = 0; n < NC; ++n) {
                            S[ii][n] = fmaf(wv, S[ii][n], fmaf(-av, us[n], kv * v[n]));
                            acc[n]   = fmaf(S[ii][n], qv, acc[n]);
                        }
                    }
                }
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    acc[n] = reduce_rg(acc[n]);
                }
                if (rg == (t & (RG - 1))) {
                    store_out(t0 + t, acc);
                }
            }
        }
        if (more) {
            park(t0 + tb, buf ^ 1);  // (the other buffer's readers passed the barrier that closed the previous stage)
        }
        __syncthreads();
    }
    if (wave_on) {
#pragma unroll
        for (int ii = 0; ii < DQ; ++ii) {
            if (ii < dq) {
#pragma unroll
                for (int n = 0; n < NC; ++n) {
                    slab[(ii * NC + n) * 64 + lane] = S[ii][n];
                }
            }
        }
    }
}

template<bool DELTA>
static void launch_state_dq(const StateMixParams& p, dim3 grid, hipStream_t st)
{
    const int  dp  = (p.dim + 7) / 8 * 8;
    auto       lds = [&](int tb) { return (2 * (size_t)tb * ((DELTA ? 5 : 2) * dp + 4 * kStateCW * kStateNC) + (DELTA ? 0 : tb * tb)) * sizeof(float); };
    const bool one = p.max_q_len == 1;  // decoded tokens: one token per stage
#define TM_STATE_LAUNCH_TB(DQ_, TB_)                                                     \
    if (p.dim == 8 * DQ_) {                                                              \
        state_mix_kernel<DQ_, DELTA, TB_, true><<<grid, 256, lds(TB_), st>>>(p);         \
    }                                                                                    \
    else {                                                                               \
        state_mix_kernel<DQ_, DELTA, TB_, false><<<grid, 256, lds(TB_), st>>>(p);        \
    }
#define TM_STATE_LAUNCH(DQ_, TB_)           \
    if (one) {                              \
        TM_STATE_LAUNCH_TB(DQ_, 1)          \
    }                                       \
    else {                                  \
        TM_STATE_LAUNCH_TB(DQ_, TB_)        \
    }
    const int dq = dp / 8;
    if (dq <= 4) {
        TM_STATE_LAUNCH(4, 16)
    }
    else if (dq <= 8) {
        TM_STATE_LAUNCH(8, 16)
    }
    else if (dq <= 16) {
        TM_STATE_LAUNCH(16, (DELTA ? 8 : 16))
    }
    else {
        TM_STATE_LAUNCH(32, (DELTA ? 4 : 8))
    }
#undef TM_STATE_LAUNCH
#undef TM_STATE_LAUNCH_TB
}

int launch_state_mix(const StateMixParams& p, bool delta, hipStream_t st)
{
    TM_REQUIRE(p.nseq >= 0 && p.heads >= 1 && p.dim >= 1 && p.dim <= 256 && p.vdim >= 1 && p.max_q_len >= 1, "state mixer: sizes (dim <= 256)");
    TM_REQUIRE(p.cu_q && p.k_len && p.state && p.proj && p.out && p.ld >= 1 && p.ldo >= p.heads * p.vdim, "state mixer: operands");
    TM_REQUIRE(delta ? (p.decay_w && p.unit && p.ld_w >= p.heads * p.dim && p.ld_u >= p.heads * p.dim) : p.decay_h != nullptr,
               "state mixer: decay operands");
    if (p.nseq == 0) {
        return 0;
    }
    const int  wcols = 4 * kStateCW * kStateNC;  // value columns of a workgroup
    const dim3 grid(p.nseq, p.heads, (p.vdim + wcols - 1) / wcols);
    if (delta) {
        launch_state_dq<true>(p, grid, st);
    }
    else {
        launch_state_dq<false>(p, grid, st);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// delta rule, per (row, head): the fused projection's key, removal-rate logits and the decay logits become what the recurrence reads --
//   unit[row][h d]  = u = k / sqrt(sum k^2 + 1e-6)
//   proj[.. c_a ..] = sigmoid(logit) * u            (in place)
//   decay[row][h d] = exp(-e^(-1/2) sigmoid(logit)) (in place)
__global__ __launch_bounds__(256) void delta_prep_kernel(float* __restrict__ proj, int ld, int c_k, int c_a, float* __restrict__ decay, int ld_w,
                                                         float* __restrict__ unit, int ld_u, int H, int D)
{
    const int t = blockIdx.x, h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= H) {
        return;
    }
    float*       pr = proj + (size_t)t * ld;
    const float* k  = pr + c_k + h * D;
    float        ss = 0.f;
    for (int i = lane; i < D; i += 64) {
        ss = fmaf(k[i], k[i], ss);
    }
    const float inv = 1.0f / sqrtf(group_sum<64>(ss) + 1e-6f);
    for (int i = lane; i < D; i += 64) {
        const float u  = k[i] * inv;
        float&      a  = pr[c_a + h * D + i];
        float&      w  = decay[(size_t)t * ld_w + h * D + i];
        a              = u / (1.f + expf(-a));
        w              = expf(-0.60653065971263342f / (1.f + expf(-w)));
        unit[(size_t)t * ld_u + h * D + i] = u;
    }
}

int launch_delta_prep(float* proj, int ld, int c_k, int c_a, float* decay, int ld_w, float* unit, int ld_u, int rows, int heads, int dim,
                      hipStream_t st)
{
    TM_REQUIRE(proj && decay && unit && heads >= 1 && dim >= 1, "delta prep: operands");
    if (rows == 0) {
        return 0;
    }
    delta_prep_kernel<<<dim3(rows, (heads + 3) / 4), 256, 0, st>>>(proj, ld, c_k, c_a, decay, ld_w, unit, ld_u, heads, dim);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// gated delta rule: one wave per (row, head) turns the convolved queries / keys and the decay logits into the vectors of the recurrence
__global__ __launch_bounds__(256) void gdelta_prep_kernel(float* __restrict__ src, int ld, int c_q, int c_k, int c_qo, int c_ko,
                                                          const float* __restrict__ beta_logit, int ld_b, float* __restrict__ decay, int ld_w,
                                                          const float* __restrict__ a_log, const float* __restrict__ dt_bias,
                                                          float* __restrict__ unit, int ld_u, int H, int G, int D)
{
    const int t = blockIdx.x, h = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (h >= H) {
        return;
    }
    const int    c  = h / (H / G);
    float*       pr = src + (size_t)t * ld;
    const float *q = pr + c_q + c * D, *k = pr + c_k + c * D;
    float        sq = 0.f, sk = 0.f;
    for (int i = lane; i < D; i += 64) {
        sq = fmaf(q[i], q[i], sq);
        sk = fmaf(k[i], k[i], sk);
    }
    const float qinv = 1.0f / (sqrtf(group_sum<64>(sq) + 1e-6f) * sqrtf((float)D));
    const float kinv = 1.0f / sqrtf(group_sum<64>(sk) + 1e-6f);
    const float beta = 1.f / (1.f + expf(-beta_logit[(size_t)t * ld_b + h]));
    const float A    = expf(a_log[h]);
    for (int i = lane; i < D; i += 64) {
        const float ku = k[i] * kinv;
        float&      w  = decay[(size_t)t * ld_w + h * D + i];
        const float z  = w + (dt_bias ? dt_bias[h * D + i] : 0.f);
        const float g  = expf(-A * (z > 20.f ? z : log1pf(expf(z))));
        w                                  = g;
        pr[c_qo + h * D + i]               = q[i] * qinv;
        pr[c_ko + h * D + i]               = beta * ku;
        unit[(size_t)t * ld_u + h * D + i] = g * ku;
    }
}

int launch_gdelta_prep(float* src, int ld, int c_q, int c_k, int c_qo, int c_ko, const float* beta_logit, int ld_b, float* decay, int ld_w,
                       const float* a_log, const float* dt_bias, float* unit, int ld_u, int rows, int heads, int kv_heads, int dim, hipStream_t st)
{
    TM_REQUIRE(src && beta_logit && decay && a_log && unit && heads >= 1 && kv_heads >= 1 && heads % kv_heads == 0 && dim >= 1, "gdelta prep: operands");
    TM_REQUIRE(c_qo >= c_q + kv_heads * dim && c_qo >= c_k + kv_heads * dim && c_ko >= c_qo + heads * dim && ld >= c_ko + heads * dim,
               "gdelta prep: the per-head vectors lie behind the convolved ones");
    if (rows == 0) {
        return 0;
    }
    gdelta_prep_kernel<<<dim3(rows, (heads + 3) / 4), 256, 0, st>>>(src, ld, c_q, c_k, c_qo, c_ko, beta_logit, ld_b, decay, ld_w, a_log, dt_bias, unit,
                                                                    ld_u, heads, kv_heads, dim);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// short causal convolution: thread = (sequence, channel, segment of kConvSeg rows); it keeps the last taps - 1 inputs in registers, so every
// input is read once.  A segment's first rows read the rows before it from x (x is not written: the output goes elsewhere) or, before the
// launch's first row, from the sequence's state; the thread of segment 0 then stores the state's new content -- nobody else touches it.
// MT: register window, taps <= MT; weights are right-aligned in it (unused taps weigh zero)
constexpr int kConvSeg = 64;

template<int MT>
__global__ __launch_bounds__(256) void short_conv_kernel(float* __restrict__ y, int ldy, const float* __restrict__ x, int ldx, int x_col,
                                                         const float* __restrict__ w, int C, int taps, int act, StateMixParams p)
{
    const int s = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x, seg = blockIdx.z;
    const int row0 = p.cu_q[s] - p.cu_q[0], q_len = p.cu_q[s + 1] - p.cu_q[s];
    const int t0 = seg * kConvSeg, t1 = min(q_len, t0 + kConvSeg);
    if (c >= C || (t0 >= q_len && seg > 0)) {
        return;
    }
    const int pos0 = p.k_len[s] - q_len, nh = taps - 1;
    int       slot = p.seq_slot ? p.seq_slot[s] : p.slot0 + s;
    if (p.active && !p.active[s]) {
        slot = p.park_slot;
    }
    float* st = p.state + (size_t)slot * p.slot_stride + p.layer_offset;  // [taps - 1][C]
    // input at row t of the launch's rows of this sequence (t < 0: history)
    auto input = [&](int t) -> float {
        if (t >= 0) {
            return x[(size_t)(row0 + t) * ldx + x_col + c];
        }
        return (pos0 > 0 && t + nh >= 0) ? st[(size_t)(t + nh) * C + c] : 0.f;
    };
    float wt[MT], win[MT - 1];
#pragma unroll
    for (int k = 0; k < MT; ++k) {
        const int j = k - (MT - taps);  // tap index
        wt[k]       = j >= 0 ? w[(size_t)c * taps + j] : 0.f;
    }
#pragma unroll
    for (int k = 0; k < MT - 1; ++k) {
        const int j = k - (MT - 1 - nh);  // history index 0 .. nh - 1, oldest first
        win[k]      = j >= 0 ? input(t0 - nh + j) : 0.f;
    }
    for (int t = t0; t < t1; ++t) {
        const float u   = x[(size_t)(row0 + t) * ldx + x_col + c];
        float       acc = 0.f;
#pragma unroll
        for (int k = 0; k < MT - 1; ++k) {
            acc = fmaf(wt[k], win[k], acc);
        }
        acc = fmaf(wt[MT - 1], u, acc);
#pragma unroll
        for (int k = 0; k + 1 < MT - 1; ++k) {
            win[k] = win[k + 1];
        }
        if (MT > 1) {
            win[MT - 2] = u;
        }
        y[(size_t)(row0 + t) * ldy + c] = act == 1 ? sm_silu(acc) : acc;
    }
    if (seg == 0) {  // new state: the inputs q_len - nh .. q_len - 1; ascending j reads st behind what it has written
        for (int j = 0; j < nh; ++j) {
            st[(size_t)j * C + c] = input(q_len - nh + j);
        }
    }
}

int launch_short_conv(float* y, int ldy, const float* x, int ldx, int x_col, const float* w, int channels, int taps, int act,
                      const StateMixParams& p, hipStream_t st)
{
    TM_REQUIRE(y && x && w && channels >= 1 && ldy >= channels && ldx >= x_col + channels && taps >= 1 && taps <= 16, "short conv: operands (1 <= taps <= 16)");
    TM_REQUIRE(p.cu_q && p.k_len && (taps == 1 || p.state) && p.max_q_len >= 1, "short conv: sequences / state");
    if (p.nseq == 0) {
        return 0;
    }
    const dim3 grid(p.nseq, (channels + 255) / 256, (p.max_q_len + kConvSeg - 1) / kConvSeg);
    if (taps <= 4) {
        short_conv_kernel<4><<<grid, 256, 0, st>>>(y, ldy, x, ldx, x_col, w, channels, taps, act, p);
    }
    else if (taps <= 8) {
        short_conv_kernel<8><<<grid, 256, 0, st>>>(y, ldy, x, ldx, x_col, w, channels, taps, act, p);
    }
    else {
        short_conv_kernel<16><<<grid, 256, 0, st>>>(y, ldy, x, ldx, x_col, w, channels, taps, act, p);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// y[row][g * n + i] = x[row][g * n + i] / sqrt(mean_i(x[row][g, :]^2) + eps) * w[g * n + i] * sigmoid(gate[row][g * n + i]):
// the output norm of the state mixers over groups of n channels (all heads together, or head by head) and their sigmoid gate.
// One workgroup per row: a single group is reduced by the whole workgroup, several groups are dealt to its four waves.
template<class T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(T* __restrict__ y, int ldy, const float* __restrict__ x, int ldx,
                                                               const float* __restrict__ w, const float* __restrict__ gate, int ldg, int groups,
                                                               int n, float eps)
{
    __shared__ float red[4];
    const int    t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float* xr = x + (size_t)t * ldx;
    if (groups == 1) {
        float ss = 0.f;
        for (int i = threadIdx.x; i < n; i += 256) {
            ss = fmaf(xr[i], xr[i], ss);
        }
        ss = group_sum<64>(ss);
        if (lane == 0) {
            red[wave] = ss;
        }
        __syncthreads();
        const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
        for (int i = threadIdx.x; i < n; i += 256) {
            y[(size_t)t * ldy + i] = (T)(xr[i] * inv * w[i] / (1.f + expf(-gate[(size_t)t * ldg + i])));
        }
        return;
    }
    for (int g = wave; g < groups; g += 4) {
        const float* xg = xr + (size_t)g * n;
        float        ss = 0.f;
        for (int i = lane; i < n; i += 64) {
            ss = fmaf(xg[i], xg[i], ss);
        }
        const float inv = 1.0f / sqrtf(group_sum<64>(ss) / (float)n + eps);
        for (int i = lane; i < n; i += 64) {
            const size_t c = (size_t)g * n + i;
            y[(size_t)t * ldy + c] = (T)(xg[i] * inv * w[c] / (1.f + expf(-gate[(size_t)t * ldg + c])));
        }
    }
}

int launch_gated_group_norm(void* y, int ldy, int out_elem_bytes, const float* x, int ldx, const float* w, const float* gate, int ldg, int rows,
                            int groups, int n, float eps, hipStream_t st)
{
    TM_REQUIRE(y && x && w && gate && groups >= 1 && n >= 1 && ldy >= groups * n && ldx >= groups * n && ldg >= groups * n, "gated norm: operands");
    if (rows == 0) {
        return 0;
    }
    if (out_elem_bytes == 2) {
        gated_group_norm_kernel<__bf16><<<rows, 256, 0, st>>>((__bf16*)y, ldy, x, ldx, w, gate, ldg, groups, n, eps);
    }
    else {
        gated_group_norm_kernel<float><<<rows, 256, 0, st>>>((float*)y, ldy, x, ldx, w, gate, ldg, groups, n, eps);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace tmk
