// Mixers with a recurrent state instead of a key / value cache: per head a matrix S [dim][vdim] in fp32 that every token updates.
//
//   linear attention ("lightning"):  S <- decay[head] S + k v^T                         o = S^T q      q, k, v = silu(projection)
//   generalized delta rule:          S <- diag(w) S - (a u)(u^T S) + k v^T              o = S^T r      u = k / sqrt(|k|^2 + 1e-6),
//                                    w, a per key channel (both terms read the old S)
//
// State pool: one state per (slot, layer run) -- slot = the engine's batch slot of the sequence, plus one parking slot for the decode
// rows of slots that hold no running sequence.  A sequence whose first row of a launch has position 0 starts from zero whatever the
// slot holds (slots are reused without clearing).  Everything here is fp32 in both number formats of the engine.
//
// The columns of S evolve independently (S[:, j] only meets v[j]), so the work is split over (sequence, head, 16 value columns): one wave
// owns a [dim][16] slab -- lane = (column c = lane % 16, row group rg = lane / 16), rows rg * dq + ii, dq = ceil(dim / 4), DQ registers --
// and walks the sequence's rows of this launch in order; the reductions over the key channels are a register sum + two lane shuffles.
// Four waves (64 value columns) share a workgroup and the LDS stage of the per-token vectors (q, k, and w, a u, u for the delta rule),
// loaded TB tokens at a time.  A slab is stored as the wave holds it, [ii][lane]: loading and storing it are fully coalesced.
// One kernel serves prompt portions (many rows per sequence) and decoded tokens (one row): the state traffic of a decode step,
// 2 * dim * vdim * 4 bytes per head, is what bounds it.
#include "tm_kernels.h"

namespace tmk {

constexpr int kStateTB = 8;  // tokens per LDS stage

__device__ __forceinline__ float sm_silu(float z)
{
    return z / (1.f + expf(-z));
}

size_t state_mix_floats(int heads, int dim, int vdim)
{
    return (size_t)heads * ((vdim + 15) / 16) * ((dim + 3) / 4) * 64;
}

// grid (nseq, heads, ceil(vdim / 64)), 256 threads, dynamic LDS = kStateTB * (NV * dim + 64) floats (NV = 2 | 5 staged vectors per token)
template<int DQ, bool DELTA>
__global__ __launch_bounds__(256) void state_mix_kernel(StateMixParams p)
{
    extern __shared__ float lds[];
    constexpr int NV = DELTA ? 5 : 2;
    const int s = blockIdx.x, h = blockIdx.y, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int D = p.dim, V = p.vdim, dq = (D + 3) / 4, ncb = (V + 15) / 16;
    const int cb = blockIdx.z * 4 + wave, c = lane & 15, rg = lane >> 4, j = cb * 16 + c;
    const bool wave_on = cb < ncb, col_on = wave_on && j < V;
    const int row0 = p.cu_q[s] - p.cu_q[0], q_len = p.cu_q[s + 1] - p.cu_q[s];
    const int pos0 = p.k_len[s] - q_len;
    int       slot = p.seq_slot ? p.seq_slot[s] : p.slot0 + s;
    if (p.active && !p.active[s]) {
        slot = p.park_slot;
    }
    float* slab = p.state + (size_t)slot * p.slot_stride + p.layer_offset + ((size_t)h * ncb + (wave_on ? cb : 0)) * dq * 64;
    float  S[DQ];
#pragma unroll
    for (int ii = 0; ii < DQ; ++ii) {
        S[ii] = (wave_on && pos0 > 0 && ii < dq) ? slab[ii * 64 + lane] : 0.f;
    }
    const float decay = DELTA ? 0.f : p.decay_h[h];
    float*      sv    = lds + (size_t)kStateTB * NV * D;  // [TB][64] values of the workgroup's columns
    for (int t0 = 0; t0 < q_len; t0 += kStateTB) {
        const int nt = min(kStateTB, q_len - t0);
        __syncthreads();
        for (int i = threadIdx.x; i < nt * D; i += 256) {
            const int    t = i / D, d = i % D;
            const size_t r = (size_t)(row0 + t0 + t);
            if constexpr (DELTA) {
                lds[(t * NV + 0) * D + d] = p.proj[r * p.ld + p.c_q + h * D + d];
                lds[(t * NV + 1) * D + d] = p.proj[r * p.ld + p.c_k + h * D + d];
                lds[(t * NV + 2) * D + d] = p.decay_w[r * p.ld_w + h * D + d];
                lds[(t * NV + 3) * D + d] = p.proj[r * p.ld + p.c_a + h * D + d];
                lds[(t * NV + 4) * D + d] = p.unit[r * p.ld_u + h * D + d];
            }
            else {
                lds[(t * NV + 0) * D + d] = sm_silu(p.proj[r * p.ld + p.c_q + h * D + d]);
                lds[(t * NV + 1) * D + d] = sm_silu(p.proj[r * p.ld + p.c_k + h * D + d]);
            }
        }
        for (int i = threadIdx.x; i < nt * 64; i += 256) {
            const int t = i >> 6, jj = blockIdx.z * 64 + (i & 63);
            float     v = 0.f;
            if (jj < V) {
                v = p.proj[(size_t)(row0 + t0 + t) * p.ld + p.c_v + h * V + jj];
                v = DELTA ? v : sm_silu(v);
            }
            sv[i] = v;
        }
        __syncthreads();
        if (!wave_on) {
            continue;
        }
        for (int t = 0; t < nt; ++t) {
            const float* q = lds + (size_t)(t * NV + 0) * D + rg * dq;
            const float* k = lds + (size_t)(t * NV + 1) * D + rg * dq;
            const float  v = sv[t * 64 + wave * 16 + c];
            float        acc = 0.f;
            if constexpr (DELTA) {
                const float* w  = lds + (size_t)(t * NV + 2) * D + rg * dq;
                const float* au = lds + (size_t)(t * NV + 3) * D + rg * dq;
                const float* u  = lds + (size_t)(t * NV + 4) * D + rg * dq;
                float        us = 0.f;
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
                    if (ii < dq && rg * dq + ii < D) {
                        us = fmaf(u[ii], S[ii], us);
                    }
                }
                us += __shfl_xor(us, 16);
                us += __shfl_xor(us, 32);
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
                    if (ii < dq && rg * dq + ii < D) {
                        S[ii] = fmaf(w[ii], S[ii], fmaf(-au[ii], us, k[ii] * v));
                        acc   = fmaf(S[ii], q[ii], acc);
                    }
                }
            }
            else {
#pragma unroll
                for (int ii = 0; ii < DQ; ++ii) {
                    if (ii < dq && rg * dq + ii < D) {
                        S[ii] = fmaf(decay, S[ii], k[ii] * v);
                        acc   = fmaf(S[ii], q[ii], acc);
                    }
                }
            }
            acc += __shfl_xor(acc, 16);
            acc += __shfl_xor(acc, 32);
            if (rg == 0 && col_on) {
                p.out[(size_t)(row0 + t0 + t) * p.ldo + h * V + j] = acc;
            }
        }
    }
    if (wave_on) {
#pragma unroll
        for (int ii = 0; ii < DQ; ++ii) {
            if (ii < dq) {
                slab[ii * 64 + lane] = S[ii];
            }
        }
    }
}

template<bool DELTA>
static void launch_state_dq(const StateMixParams& p, dim3 grid, size_t lds, hipStream_t st)
{
    const int dq = (p.dim + 3) / 4;
    if (dq <= 8) {
        state_mix_kernel<8, DELTA><<<grid, 256, lds, st>>>(p);
    }
    else if (dq <= 16) {
        state_mix_kernel<16, DELTA><<<grid, 256, lds, st>>>(p);
    }
    else if (dq <= 32) {
        state_mix_kernel<32, DELTA><<<grid, 256, lds, st>>>(p);
    }
    else {
        state_mix_kernel<64, DELTA><<<grid, 256, lds, st>>>(p);
    }
}

int launch_state_mix(const StateMixParams& p, bool delta, hipStream_t st)
{
    TM_REQUIRE(p.nseq >= 0 && p.heads >= 1 && p.dim >= 1 && p.dim <= 256 && p.vdim >= 1, "state mixer: sizes (dim <= 256)");
    TM_REQUIRE(p.cu_q && p.k_len && p.state && p.proj && p.out && p.ld >= 1 && p.ldo >= p.heads * p.vdim, "state mixer: operands");
    TM_REQUIRE(delta ? (p.decay_w && p.unit && p.ld_w >= p.heads * p.dim && p.ld_u >= p.heads * p.dim && p.vdim == p.dim) : p.decay_h != nullptr,
               "state mixer: decay operands");
    if (p.nseq == 0) {
        return 0;
    }
    const dim3   grid(p.nseq, p.heads, (p.vdim + 63) / 64);
    const size_t lds = (size_t)kStateTB * ((delta ? 5 : 2) * p.dim + 64) * sizeof(float);
    if (delta) {
        launch_state_dq<true>(p, grid, lds, st);
    }
    else {
        launch_state_dq<false>(p, grid, lds, st);
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

// y[row][g * n + i] = x[row][g * n + i] / sqrt(mean_i(x[row][g, :]^2) + eps) * w[g * n + i] * sigmoid(gate[row][g * n + i]):
// the output norm of the state mixers over groups of n channels (all heads together, or head by head) and their sigmoid gate.
// grid (rows, groups), 256 threads
template<class T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(T* __restrict__ y, int ldy, const float* __restrict__ x, int ldx,
                                                               const float* __restrict__ w, const float* __restrict__ gate, int ldg, int n,
                                                               float eps)
{
    __shared__ float red[4];
    const int    t = blockIdx.x, g = blockIdx.y;
    const float* xr = x + (size_t)t * ldx + (size_t)g * n;
    float        ss = 0.f;
    for (int i = threadIdx.x; i < n; i += 256) {
        ss = fmaf(xr[i], xr[i], ss);
    }
    ss = group_sum<64>(ss);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = ss;
    }
    __syncthreads();
    const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)n + eps);
    for (int i = threadIdx.x; i < n; i += 256) {
        const size_t c = (size_t)g * n + i;
        const float  z = gate[(size_t)t * ldg + c];
        y[(size_t)t * ldy + c] = (T)(xr[i] * inv * w[c] / (1.f + expf(-z)));
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
        gated_group_norm_kernel<__bf16><<<dim3(rows, groups), 256, 0, st>>>((__bf16*)y, ldy, x, ldx, w, gate, ldg, n, eps);
    }
    else {
        gated_group_norm_kernel<float><<<dim3(rows, groups), 256, 0, st>>>((float*)y, ldy, x, ldx, w, gate, ldg, n, eps);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace tmk
