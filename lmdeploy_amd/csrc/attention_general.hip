// Paged causal attention for arbitrary head sizes (key size `dim`, value size `vdim`, grouped query heads), bf16 or fp32 cache,
// with the score modifiers of recent decoder designs as PARAMETERS (GeneralAttnParams), each off at its neutral value:
//   * query temperature by position: score *= 1 + coef * ln(floor((p + 1) / every) + 1)          (coef = 0: off)
//   * soft cap:                      score  = cap * tanh(score / cap)                               (cap <= 0: off)
//   * attention sink:                the softmax denominator also holds exp(sink[head]): a learned logit with no key and no value,
//                                    neither scaled nor capped                                      (sink = nullptr: off)
//   * distance penalty:              score -= r1[head] * ln(1 + r2[head] * (p - key position))      (dist_r1 = nullptr: off)
//   * chunked visibility:            a row sees the keys of its own chunk of positions only:
//                                    key >= floor(p / chunk) * chunk, chunks counted from position 0   (chunk = 0: off)
//   * output gate:                   head h of row t is multiplied by sigmoid(out_gate[t][h])        (out_gate = nullptr: off)
//   * sliding window:                a row at position p sees key j <= p only if p - j < window or j < keep_first: the window plus
//                                    the first tokens of the sequence, at their true positions             (window = 0: off)
//   * distance table:                score += dist_table[head][min(p - key position, len - 1)]: a learned bias per distance (a bucketed
//                                    table is expanded per distance by the caller)                   (dist_table = nullptr: off)
//   * key / value head counts of their own: the query heads form kv_heads groups; group g reads key head g % k_heads and value head
//                                    g % v_heads (two score maps over one set of values; one wide key with a value head per group)
// Scores, soft-max weights and the output accumulation are fp32 whatever the cache holds; out_f32 keeps the output rows in fp32 too.
//
// One launch serves every row of a forward, prefill portions and decoded tokens alike: row t belongs to sequence row_seq[t] at
// position row_pos[t] and sees the cache entries 0 .. row_pos[t] of that sequence (its own key was stored before the launch).
//   * row kernel : one wave per (row, query head, key split); lanes own keys for the scores and value channels for the output.
//                  The decode path (few rows, long contexts: split keys + merge kernel) and the fp32 path.
//   * tile kernel: bf16 prefill on the matrix cores -- 64 query rows of one sequence x one query head per workgroup, four waves of 16
//                  rows; S^T = K Q^T and O^T += V^T P^T as v_mfma_f32_16x16x32_bf16 with every operand a 16-byte load straight from the
//                  cache (keys [token][channel], values stored transposed [channel][token]); online soft-max in fp32; no LDS, no barrier.
//   * decode kernel: the same products with the query HEADS of one key head as the 16 rows (one row per sequence): a workgroup per
//                  (sequence, key head, key split), its four waves take every fourth cache block and merge at the end.
// Cache block layout per layer: keys [kv_heads][64][dim], then values [kv_heads][vdim][64].
#include "tm_kernels.h"
#include <stdlib.h>

#define TM_TRY_RC(expr)      \
    do {                     \
        int _rc = (expr);    \
        if (_rc) {           \
            return _rc;      \
        }                    \
    } while (0)

namespace tmk {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float ga_wave_max(float v)
{
    return group_max<64>(v);
}
__device__ __forceinline__ float ga_wave_sum(float v)
{
    return group_sum<64>(v);
}

__device__ __forceinline__ float ga_query_temp(const GeneralAttnParams& p, int pos)
{
    if (p.qtemp_coef == 0.f) {
        return 1.f;
    }
    const float steps = (float)floor((double)(pos + 1) / (double)p.qtemp_every);
    return 1.f + p.qtemp_coef * logf(steps + 1.f);
}

__device__ __forceinline__ float ga_modify(const GeneralAttnParams& p, float dot, float qscale)
{
    float s = dot * qscale;
    if (p.softcap > 0.f) {
        s = p.softcap * tanhf(s / p.softcap);
    }
    return s;
}

template<class T>
__device__ __forceinline__ float ga_dot(const T* __restrict__ k, const float* __restrict__ q, int D)
{
    float acc = 0.f;
    if constexpr (sizeof(T) == 2) {
        if ((D & 7) == 0) {
            for (int d = 0; d < D; d += 8) {
                const bf16x8 v = *(const bf16x8*)(k + d);
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    acc = fmaf((float)v[i], q[d + i], acc);
                }
            }
            return acc;
        }
    }
    else {
        if ((D & 3) == 0) {
            for (int d = 0; d < D; d += 4) {
                const floatx4 v = *(const floatx4*)(k + d);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc = fmaf(v[i], q[d + i], acc);
                }
            }
            return acc;
        }
    }
    for (int d = 0; d < D; ++d) {
        acc = fmaf((float)k[d], q[d], acc);
    }
    return acc;
}

constexpr int kGaMaxDim = 1024;  // key size limit of the row kernel (q in LDS); value size: 64 * VC, VC value channels per lane

// first key of the contiguous range a row sees (its chunk's first position, or the window's)
__device__ __forceinline__ int ga_first_key(const GeneralAttnParams& p, int pos)
{
    const int f = p.chunk > 0 ? pos / p.chunk * p.chunk : 0;
    return p.window > 0 ? max(f, pos - p.window + 1) : f;
}
// keys below that range stay visible while they are among the first ga_keep() positions.  The blocks a row visits are then the
// `nk` blocks that hold such keys and lie before the range's first block `bf`, followed by bf .. (last block): ga_block_at maps an index of
// that list to the block; key splits divide the list.
__device__ __forceinline__ int ga_keep(const GeneralAttnParams& p)
{
    return p.window > 0 ? p.keep_first : 0;
}
__device__ __forceinline__ int ga_keep_blocks(const GeneralAttnParams& p, int first, int bf, int block_len)
{
    return min(bf, (min(ga_keep(p), first) + block_len - 1) / block_len);
}
__device__ __forceinline__ int ga_block_at(int bi, int nk, int bf)
{
    return bi < nk ? bi : bf + (bi - nk);
}

// where head h of an output row starts: heads side by side unless the caller spaces them (a batched product reads them at a stride)
__device__ __forceinline__ size_t ga_out_head(const GeneralAttnParams& p, int h)
{
    return (size_t)h * (p.out_head_stride > 0 ? p.out_head_stride : p.vdim);
}

__device__ __forceinline__ float ga_out_gate(const GeneralAttnParams& p, int t, int h)
{
    return p.out_gate ? 1.f / (1.f + expf(-p.out_gate[(size_t)t * p.ld_gate + h])) : 1.f;
}

// key / value head of a group of query heads
__device__ __forceinline__ int ga_key_head(const GeneralAttnParams& p, int g)
{
    return p.k_heads > 0 ? g % p.k_heads : g;
}
__device__ __forceinline__ int ga_value_head(const GeneralAttnParams& p, int g)
{
    return p.v_heads > 0 ? g % p.v_heads : g;
}

// channel v of head h of output row t
template<class T>
__device__ __forceinline__ void ga_store(const GeneralAttnParams& p, int t, int h, int v, float val)
{
    const size_t at = (size_t)t * p.ldo + ga_out_head(p, h) + v;
    if (p.out_f32) {
        ((float*)p.out)[at] = val;
    }
    else {
        ((T*)p.out)[at] = (T)val;
    }
}

// grid (rows, ceil(q_heads / 4), splits), 256 threads: wave w -> head blockIdx.y * 4 + w
template<class T, int VC>
__global__ __launch_bounds__(256) void attn_rows_kernel(GeneralAttnParams p)
{
    __shared__ float qs[4][kGaMaxDim];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x, h = blockIdx.y * 4 + wave, sp = blockIdx.z;
    if (h >= p.q_heads) {
        return;
    }
    const int D = p.dim, V = p.vdim;
    const int s = p.row_seq[t], pos = p.row_pos[t];
    const int g = h / (p.q_heads / p.kv_heads);
    const uint64_t* table = p.block_ptrs + (size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride;
    const T* q = (const T*)p.q + (size_t)t * p.ldq + (size_t)h * D;
    for (int d = lane; d < D; d += 64) {
        qs[wave][d] = (float)q[d];
    }
    const float qscale = p.scale * ga_query_temp(p, pos);
    const int   nkeys = pos + 1, nblk = (nkeys + p.block_len - 1) / p.block_len;
    const int   first = ga_first_key(p, pos), bf = first / p.block_len;  // the first key of the visible range and its block
    const int   keep = ga_keep(p), nk = ga_keep_blocks(p, first, bf, p.block_len), nvis = nk + nblk - bf;
    const int   per = (nvis + p.splits - 1) / p.splits;
    const int   i0 = sp * per, i1 = min(nvis, i0 + per);
    const float r1 = p.dist_r1 ? p.dist_r1[h] : 0.f, r2 = p.dist_r1 ? p.dist_r2[h] : 0.f;
    float m = -1e30f, l = 0.f, o[VC];
#pragma unroll
    for (int c = 0; c < VC; ++c) {
        o[c] = 0.f;
    }
    // LDS writes of this wave are read by this wave only: a wave barrier is enough
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int bi = i0; bi < i1; ++bi) {
        const int   b    = ga_block_at(bi, nk, bf);
        const char* base = (const char*)table[b] + p.layer_offset;
        const T*    kb   = (const T*)base + (size_t)ga_key_head(p, g) * p.block_len * D;
        const T*    vb   = (const T*)(base + p.v_offset) + (size_t)ga_value_head(p, g) * p.block_len * V;  // [V][block_len]
        const int   n    = min(p.block_len, nkeys - b * p.block_len);
        const int   jlo  = first - b * p.block_len;  // keys below it lie in an earlier chunk / before the window ...
        const int   klo  = keep - b * p.block_len;   // ... and are seen only as kept first tokens: j < klo
        for (int j0 = klo > 0 ? 0 : max(0, jlo) / 64 * 64; j0 < n; j0 += 64) {
            const int  j     = j0 + lane;
            const bool valid = j < n && (j >= jlo || j < klo);
            float      sc    = -1e30f;
            if (valid) {
                sc = ga_modify(p, ga_dot<T>(kb + (size_t)j * D, qs[wave], D), qscale);
                if (p.dist_r1) {
                    sc -= r1 * log1pf(r2 * (float)(pos - (b * p.block_len + j)));
                }
                if (p.dist_table) {
                    sc += p.dist_table[(size_t)h * p.dist_table_len + min(pos - (b * p.block_len + j), p.dist_table_len - 1)];
                }
            }
            const float m_new = fmaxf(m, ga_wave_max(sc));
            const float alpha = __expf(m - m_new);
            const float pj    = valid ? __expf(sc - m_new) : 0.f;
            l                 = l * alpha + ga_wave_sum(pj);
            m                 = m_new;
#pragma unroll
            for (int c = 0; c < VC; ++c) {
                o[c] *= alpha;
            }
            const int cnt = min(64, n - j0);
            for (int jj = klo > 0 ? 0 : max(0, jlo - j0); jj < cnt; ++jj) {
                const float w  = __shfl(pj, jj);
                const T*    vr = vb + (j0 + jj);
#pragma unroll
                for (int c = 0; c < VC; ++c) {
                    const int v = lane + 64 * c;
                    if (v < V) {
                        o[c] = fmaf(w, (float)vr[(size_t)v * p.block_len], o[c]);
                    }
                }
            }
        }
    }
    if (p.splits == 1) {
        float inv;
        if (p.sink) {
            const float sk = p.sink[h], mf = fmaxf(m, sk), a = __expf(m - mf);
            inv            = a / (l * a + __expf(sk - mf));
        }
        else {
            inv = 1.f / l;
        }
        inv *= ga_out_gate(p, t, h);
#pragma unroll
        for (int c = 0; c < VC; ++c) {
            const int v = lane + 64 * c;
            if (v < V) {
                ga_store<T>(p, t, h, v, o[c] * inv);
            }
        }
        return;
    }
    float* po = p.partial_o + (((size_t)t * p.q_heads + h) * p.splits + sp) * V;
    float* pm = p.partial_ml + (((size_t)t * p.q_heads + h) * p.splits + sp) * 2;
#pragma unroll
    for (int c = 0; c < VC; ++c) {
        const int v = lane + 64 * c;
        if (v < V) {
            po[v] = o[c];
        }
    }
    if (lane == 0) {
        pm[0] = m;
        pm[1] = l;
    }
}

// merge of the key splits (+ the sink): grid (rows, q_heads), 64 threads
template<class T, int VC>
__global__ __launch_bounds__(64) void attn_rows_merge_kernel(GeneralAttnParams p)
{
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, V = p.vdim;
    const float* pm = p.partial_ml + ((size_t)t * p.q_heads + h) * p.splits * 2;
    const float* po = p.partial_o + ((size_t)t * p.q_heads + h) * p.splits * V;
    float        mf = p.sink ? p.sink[h] : -1e30f;
    for (int s = 0; s < p.splits; ++s) {
        mf = fmaxf(mf, pm[s * 2]);
    }
    float l = p.sink ? __expf(p.sink[h] - mf) : 0.f;
    float o[VC];
#pragma unroll
    for (int c = 0; c < VC; ++c) {
        o[c] = 0.f;
    }
    for (int s = 0; s < p.splits; ++s) {
        const float a = __expf(pm[s * 2] - mf);
        l += a * pm[s * 2 + 1];
#pragma unroll
        for (int c = 0; c < VC; ++c) {
            const int v = lane + 64 * c;
            if (v < V) {
                o[c] = fmaf(a, po[(size_t)s * V + v], o[c]);
            }
        }
    }
    const float inv = ga_out_gate(p, t, h) / l;
#pragma unroll
    for (int c = 0; c < VC; ++c) {
        const int v = lane + 64 * c;
        if (v < V) {
            ga_store<T>(p, t, h, v, o[c] * inv);
        }
    }
}

template<class T>
static void launch_rows_merge(const GeneralAttnParams& p, hipStream_t st)
{
    if (p.vdim <= 256) {
        attn_rows_merge_kernel<T, 4><<<dim3(p.rows, p.q_heads), 64, 0, st>>>(p);
    }
    else {
        attn_rows_merge_kernel<T, 16><<<dim3(p.rows, p.q_heads), 64, 0, st>>>(p);
    }
}

template<class T>
static void launch_rows(const GeneralAttnParams& p, dim3 grid, hipStream_t st)
{
    if (p.vdim <= 256) {
        attn_rows_kernel<T, 4><<<grid, 256, 0, st>>>(p);
    }
    else {
        attn_rows_kernel<T, 16><<<grid, 256, 0, st>>>(p);
    }
}

size_t general_attention_workspace_bytes(int rows, int q_heads, int vdim, int splits)
{
    return (size_t)rows * q_heads * splits * (vdim + 2) * sizeof(float);
}

int launch_general_attention_rows(const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(p.rows >= 0 && p.q_heads >= 1 && p.kv_heads >= 1 && p.q_heads % p.kv_heads == 0, "attention: head counts");
    TM_REQUIRE(p.dim >= 1 && p.dim <= kGaMaxDim && p.vdim >= 1 && p.vdim <= kGaMaxDim, "attention: 1 <= dim, vdim <= 1024");
    TM_REQUIRE(p.chunk >= 0 && (!p.dist_r1 || p.dist_r2) && (!p.out_gate || p.ld_gate >= p.q_heads), "attention: chunk / distance penalty / gate");
    TM_REQUIRE(p.window >= 0 && p.keep_first >= 0, "attention: window / kept first tokens");
    TM_REQUIRE(p.k_heads >= 0 && p.v_heads >= 0 && (!p.dist_table || p.dist_table_len >= 1), "attention: key / value head counts, distance table");
    TM_REQUIRE(p.block_len >= 1 && p.splits >= 1 && (p.splits == 1 || (p.partial_o && p.partial_ml)), "attention: splits / workspace");
    TM_REQUIRE(p.elem_bytes == 2 || p.elem_bytes == 4, "attention: bf16 or fp32");
    TM_REQUIRE(p.qtemp_coef == 0.f || p.qtemp_every > 0.f, "attention: query temperature period");
    if (p.rows == 0) {
        return 0;
    }
    const dim3 grid(p.rows, (p.q_heads + 3) / 4, p.splits);
    if (p.elem_bytes == 2) {
        launch_rows<__bf16>(p, grid, st);
    }
    else {
        launch_rows<float>(p, grid, st);
    }
    TM_HIP_CHECK(hipGetLastError());
    if (p.splits > 1) {
        if (p.elem_bytes == 2) {
            launch_rows_merge<__bf16>(p, st);
        }
        else {
            launch_rows_merge<float>(p, st);
        }
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}


// ---- matrix-core kernels (bf16) -------------------------------------------------------------------------------------------------------
// Per 64-key cache block a wave computes the TRANSPOSED scores S^T = K Q^T as four 16-key tiles (A = key rows, B = query rows; one
// 16-byte load per lane and 32 channels), so that a lane ends up with 16 scores of ONE query row (row = lane % 16): the soft-max
// statistics are per-lane scalars (two shuffles join the four lane groups) and the exponentiated accumulators ARE the B operand of
// O^T += V^T P^T.  Which 16 keys form a tile is free: tile kt, A-row i is key (kt / 2) * 32 + (i / 4) * 8 + (kt % 2) * 4 + i % 4, which
// leaves lane group lg with the EIGHT CONSECUTIVE keys ks * 32 + lg * 8 .. + 8 of k-step ks in its two tiles -- the A operand of the
// second product is then one 16-byte load from the transposed values.  No score or probability ever goes through memory.
constexpr int   kTileRows = 64;
constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;

__device__ __forceinline__ float ga_tanh_fast(float x)
{
    // 1 - 2 / (exp(2x) + 1): absolute error ~1e-7, exact limits at +-inf
    return 1.f - 2.f * __builtin_amdgcn_rcpf(__expf(2.f * x) + 1.f);
}

// one 64-key block for RT tiles of 16 query rows (the lane's row of tile rt is rt * 16 + lane % 16): updates (m, l, o) of those rows.
// Every key / value fragment is loaded ONCE and serves all RT row tiles; the value fragments are requested before the soft-max
// arithmetic so that their latency hides under it.  qf: the rows' query fragments; limit: last visible key of the lane's rows
// (block-relative; < 0: none); kb / vb: the key head's keys [64][D] and transposed values [V][64] of this block.
// lower: first key of the visible range of the lane's rows (block-relative, may be negative); keys below it are seen while < keep_rel
// (the kept first tokens, block-relative; <= 0: none); r1 / r2: the distance penalty of the lane's rows' head
// (r1 * log2(1 + r2 * (limit - key)) leaves the score, which lives in the log2 domain; bias = false: none); tab: the distance table's row
// of the lane's rows' head (nullptr: none)
template<int DS, int VT, int RT, bool MASK, bool EAGER>
__device__ __forceinline__ void ga_block_step(const bf16x8 (&qf)[RT][DS], const __bf16* __restrict__ kb, const __bf16* __restrict__ vb, int D,
                                              int V, const int (&limit)[RT], const int (&lower)[RT], int keep_rel, const float (&qscale)[RT], float cap,
                                              float inv_cap, bool bias, float r1, float r2, float (&m)[RT], float (&l)[RT],
                                              floatx4 (&o)[RT][VT], const float* __restrict__ tab = nullptr, int tab_len = 0)
{
    const int    lane = threadIdx.x & 63, lr = lane & 15, lg = lane >> 4;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    floatx4      sc[RT][4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            sc[rt][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
        const __bf16* kr = kb + (size_t)((kt >> 1) * 32 + (lr >> 2) * 8 + (kt & 1) * 4 + (lr & 3)) * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            // EAGER (decode: a wave has one or two blocks, latency is everything): every load is unconditional -- clamped address, value
            // selected afterwards -- so that all of them are in flight at once; a guarded load is waited for at the join of its branch.
            // The prefill kernel keeps the guarded form: with four row tiles per wave the eager form costs registers it does not have.
            const int d = ds * 32 + lg * 8;
            bf16x8    kf;
            if constexpr (EAGER) {
                const bf16x8 kl = *(const bf16x8*)(kr + min(d, D - 8));
                kf              = d < D ? kl : zero8;
            }
            else {
                kf = d < D ? *(const bf16x8*)(kr + d) : zero8;
            }
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                sc[rt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[rt][ds], sc[rt][kt], 0, 0, 0);
            }
        }
    }
    bf16x8 vf[VT][2];
#pragma unroll
    for (int t = 0; t < VT; ++t) {
        const int v = t * 16 + lr;
        if constexpr (EAGER) {
            const __bf16* vr = vb + (size_t)min(v, V - 1) * 64 + lg * 8;
            const bf16x8  v0 = *(const bf16x8*)(vr), v1 = *(const bf16x8*)(vr + 32);
            vf[t][0]         = v < V ? v0 : zero8;
            vf[t][1]         = v < V ? v1 : zero8;
        }
        else {
            const __bf16* vr = vb + (size_t)v * 64 + lg * 8;
            vf[t][0]         = v < V ? *(const bf16x8*)(vr) : zero8;
            vf[t][1]         = v < V ? *(const bf16x8*)(vr + 32) : zero8;
        }
    }
    // lane holds S[row lr of tile rt][key (kt / 2) * 32 + lg * 8 + (kt % 2) * 4 + r].  From here on scores live in the log2 domain
    // (multiplied by log2 e) so that every exponential is one v_exp_f32: the capped score is
    //   cap2 * tanh(x / cap) = cap2 - 2 cap2 / (2^(x * 2 log2e / cap) + 1),  cap2 = cap * log2e
    // -- five VALU operations, two of them transcendental; the kernel is bound by exactly this arithmetic.
    bf16x8 pf[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const float cap2 = cap * kLog2e, k1 = cap > 0.f ? qscale[rt] * inv_cap * (2.f * kLog2e) : qscale[rt] * kLog2e;
        float       bmax = -1e30f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = sc[rt][kt][r] * k1;
                if (cap > 0.f) {
                    v = fmaf(__builtin_amdgcn_rcpf(fast_exp2(v) + 1.f), -2.f * cap2, cap2);
                }
                const int key = (kt >> 1) * 32 + lg * 8 + (kt & 1) * 4 + r;
                if (bias) {  // (a key ahead of the row gives the logarithm of a number that may be negative: the mask below discards it)
                    v = fmaf(-r1, __builtin_amdgcn_logf(fmaf(r2, (float)(limit[rt] - key), 1.f)), v);
                }
                if (tab) {  // the lane's head's row of the distance table (a key ahead of the row reads entry 0 and is masked below)
                    v = fmaf(tab[min(max(limit[rt] - key, 0), tab_len - 1)], kLog2e, v);
                }
                if (MASK) {
                    v = (key <= limit[rt] && (key >= lower[rt] || key < keep_rel)) ? v : -1e30f;
                }
                sc[rt][kt][r] = v;
                bmax          = fmaxf(bmax, v);
            }
        }
        bmax = fmaxf(bmax, __shfl_xor(bmax, 16));
        bmax = fmaxf(bmax, __shfl_xor(bmax, 32));
        const float m_new = fmaxf(m[rt], bmax);
        const float alpha = fast_exp2(m[rt] - m_new);
        const float m_ref = fmaxf(m_new, -1e29f);  // a row that has seen no key yet (its chunk starts behind this block): every weight is 0
        float       bsum  = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float e = fast_exp2(sc[rt][kt][r] - m_ref);  // a masked score is -1e30: 2^(-1e30 - m) = 0
                bsum += e;
                pf[rt][kt >> 1][(kt & 1) * 4 + r] = (__bf16)e;
            }
        }
        bsum += __shfl_xor(bsum, 16);
        bsum += __shfl_xor(bsum, 32);
        l[rt] = l[rt] * alpha + bsum;
        m[rt] = m_new;
#pragma unroll
        for (int t = 0; t < VT; ++t) {
            o[rt][t] *= alpha;
        }
    }
#pragma unroll
    for (int t = 0; t < VT; ++t) {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                o[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[t][ks], pf[rt][ks], o[rt][t], 0, 0, 0);
            }
        }
    }
}

// Prefill: workgroup = 64 * RT query rows of one sequence x one query head, four independent waves of RT tiles of 16 rows.
template<int DS /* 32-channel steps of the key size */, int VT /* 16-channel tiles of the value size */, int RT>
__global__ __launch_bounds__(256) void attn_tiles_kernel(GeneralAttnParams p, int tiles_per_seq)
{
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int s = blockIdx.x / tiles_per_seq, ti = blockIdx.x % tiles_per_seq, h = blockIdx.y;
    const int row_base = p.cu_q[s] - p.cu_q[0];
    const int q_len = p.cu_q[s + 1] - p.cu_q[s];
    const int row0  = ti * (kTileRows * RT) + wave * (16 * RT);  // the wave's first row inside the sequence's portion
    if (row0 >= q_len) {
        return;
    }
    const int D = p.dim, V = p.vdim;
    const int g = h / (p.q_heads / p.kv_heads);
    const int pos0 = p.k_len[s] - q_len;  // position of the sequence's first row in this launch
    const int lr = lane & 15, lg = lane >> 4;
    const uint64_t* table = p.block_ptrs + (size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    const float cap = p.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
    bf16x8  qf[RT][DS];  // B operand of S^T: row = lane % 16, channels ds * 32 + (lane / 16) * 8 .. + 8
    float   qscale[RT], m[RT], l[RT];
    int     pos[RT], first[RT];
    const bool  bias = p.dist_r1 != nullptr;
    const float r1 = bias ? p.dist_r1[h] : 0.f, r2 = bias ? p.dist_r2[h] : 0.f;
    const float* tab = p.dist_table ? p.dist_table + (size_t)h * p.dist_table_len : nullptr;
    bool    q_ok[RT];
    floatx4 o[RT][VT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int qi = row0 + rt * 16 + lr;
        q_ok[rt]     = qi < q_len;
        pos[rt]      = pos0 + qi;
        first[rt]    = ga_first_key(p, pos[rt]);
        const __bf16* q = (const __bf16*)p.q + (size_t)(row_base + (q_ok[rt] ? qi : 0)) * p.ldq + (size_t)h * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int    d  = ds * 32 + lg * 8;
            const bf16x8 ql = *(const bf16x8*)(q + min(d, D - 8));
            qf[rt][ds]      = (q_ok[rt] && d < D) ? ql : zero8;
        }
        qscale[rt] = p.scale * ga_query_temp(p, pos[rt]);
        m[rt]      = -1e30f;
        l[rt]      = 0.f;
#pragma unroll
        for (int t = 0; t < VT; ++t) {
            o[rt][t] = floatx4{0.f, 0.f, 0.f, 0.f};
        }
    }
    const int last_pos = pos0 + min(q_len, row0 + 16 * RT) - 1;  // the wave's last row sees keys 0 .. last_pos
    const int nblk     = last_pos / 64 + 1;
    const int first_lo = ga_first_key(p, pos0 + row0), first_hi = ga_first_key(p, last_pos);  // of the wave's first and last row
    const int keep = ga_keep(p), bf = first_lo / 64, nk = ga_keep_blocks(p, first_lo, bf, 64);
    for (int bi = 0; bi < nk + nblk - bf; ++bi) {
        const int   b    = ga_block_at(bi, nk, bf);
        const char* base = (const char*)table[b] + p.layer_offset;
        int         limit[RT], lower[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            limit[rt] = q_ok[rt] ? pos[rt] - b * 64 : -1;
            lower[rt] = first[rt] - b * 64;
        }
        const __bf16 *kb = (const __bf16*)base + (size_t)ga_key_head(p, g) * 64 * D;
        const __bf16 *vb = (const __bf16*)(base + p.v_offset) + (size_t)ga_value_head(p, g) * 64 * V;
        // every row of the wave sees the whole block (rows beyond the portion are discarded anyway)
        if (b * 64 + 63 <= pos0 + row0 && b * 64 >= first_hi) {
            ga_block_step<DS, VT, RT, false, false>(qf, kb, vb, D, V, limit, lower, 0, qscale, cap, inv_cap, bias, r1, r2, m, l, o, tab, p.dist_table_len);
        }
        else {
            ga_block_step<DS, VT, RT, true, false>(qf, kb, vb, D, V, limit, lower, keep - b * 64, qscale, cap, inv_cap, bias, r1, r2, m, l, o, tab,
                                                   p.dist_table_len);
        }
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        if (!q_ok[rt]) {
            continue;
        }
        float inv;
        if (p.sink) {  // m is in the log2 domain
            const float sk = p.sink[h] * kLog2e, mf = fmaxf(m[rt], sk), a = fast_exp2(m[rt] - mf);
            inv            = a / (l[rt] * a + fast_exp2(sk - mf));
        }
        else {
            inv = 1.f / l[rt];
        }
        inv *= ga_out_gate(p, row_base + row0 + rt * 16 + lr, h);
        // lane holds O[row lr][channel t * 16 + lg * 4 + r]
#pragma unroll
        for (int t = 0; t < VT; ++t) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int v = t * 16 + lg * 4 + r;
                if (v < V) {
                    ga_store<__bf16>(p, row_base + row0 + rt * 16 + lr, h, v, o[rt][t][r] * inv);
                }
            }
        }
    }
}

// Decode: grid (sequences, kv_heads * head chunks, splits).  The 16 rows are query heads g * group + chunk * 16 + (lane % 16) of row t;
// wave w takes the blocks b0 + w, b0 + w + 4, ... of the split; waves 1..3 hand their (m, l, O) to wave 0 through LDS.
template<int DS, int VT>
__global__ __launch_bounds__(256) void attn_decode_kernel(GeneralAttnParams p, int chunks)
{
    __shared__ float ml_s[4][16][2];
    __shared__ float o_s[3][16][VT * 16];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int t = blockIdx.x, g = blockIdx.y / chunks, chunk = blockIdx.y % chunks, sp = blockIdx.z;
    const int D = p.dim, V = p.vdim, group = p.q_heads / p.kv_heads;
    const int lr = lane & 15, lg = lane >> 4;
    const int hg = chunk * 16 + lr;           // head inside the group
    const bool h_ok = hg < group;
    const int  h    = g * group + (h_ok ? hg : 0);
    const int  s = p.row_seq[t], pos = p.row_pos[t];
    const uint64_t* table = p.block_ptrs + (size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
    bf16x8 qf[1][DS];
    {
        const __bf16* q = (const __bf16*)p.q + (size_t)t * p.ldq + (size_t)h * D;
#pragma unroll
        for (int ds = 0; ds < DS; ++ds) {
            const int    d  = ds * 32 + lg * 8;
            const bf16x8 ql = *(const bf16x8*)(q + min(d, D - 8));
            qf[0][ds]       = (h_ok && d < D) ? ql : zero8;
        }
    }
    const float qscale[1] = {p.scale * ga_query_temp(p, pos)};
    const float cap = p.softcap, inv_cap = cap > 0.f ? 1.f / cap : 0.f;
    float   m1[1] = {-1e30f}, l1[1] = {0.f};
    floatx4 o1[1][VT];
#pragma unroll
    for (int v = 0; v < VT; ++v) {
        o1[0][v] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    const bool  bias = p.dist_r1 != nullptr;
    const float r1 = bias ? p.dist_r1[h] : 0.f, r2 = bias ? p.dist_r2[h] : 0.f;  // of the lane's head
    const float* tab = p.dist_table ? p.dist_table + (size_t)h * p.dist_table_len : nullptr;
    const int first = ga_first_key(p, pos), bf = first / 64;
    const int keep = ga_keep(p), nk = ga_keep_blocks(p, first, bf, 64);
    const int nvis = nk + pos / 64 + 1 - bf, per = (nvis + p.splits - 1) / p.splits;
    const int i0 = sp * per, i1 = min(nvis, i0 + per);
    for (int bi = i0 + wave; bi < i1; bi += 4) {
        const int   b    = ga_block_at(bi, nk, bf);
        const char* base = (const char*)table[b] + p.layer_offset;
        const int limit[1] = {pos - b * 64}, lower[1] = {first - b * 64};
        ga_block_step<DS, VT, 1, true, true>(qf, (const __bf16*)base + (size_t)ga_key_head(p, g) * 64 * D,
                                             (const __bf16*)(base + p.v_offset) + (size_t)ga_value_head(p, g) * 64 * V, D, V, limit, lower,
                                             keep - b * 64, qscale, cap, inv_cap, bias, r1, r2, m1, l1, o1, tab, p.dist_table_len);
    }
    const float m = m1[0] * kLn2, l = l1[0];  // back from the log2 domain: the merge below and the split merge kernel use e^x
    floatx4 (&o)[VT] = o1[0];
    // ---- merge the four waves: common maximum, rescaled sums ----
    if (lg == 0) {
        ml_s[wave][lr][0] = m;
        ml_s[wave][lr][1] = l;
    }
    __syncthreads();
    const float mf = fmaxf(fmaxf(ml_s[0][lr][0], ml_s[1][lr][0]), fmaxf(ml_s[2][lr][0], ml_s[3][lr][0]));
    const float a  = __expf(m - mf);
    if (wave > 0) {
#pragma unroll
        for (int v = 0; v < VT; ++v) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                o_s[wave - 1][lr][v * 16 + lg * 4 + r] = o[v][r] * a;
            }
        }
    }
    __syncthreads();
    if (wave > 0 || !h_ok) {
        return;
    }
    float lt = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        lt += ml_s[w][lr][1] * __expf(ml_s[w][lr][0] - mf);
    }
#pragma unroll
    for (int v = 0; v < VT; ++v) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int c = v * 16 + lg * 4 + r;
            o[v][r]     = o[v][r] * a + ((o_s[0][lr][c] + o_s[1][lr][c]) + o_s[2][lr][c]);
        }
    }
    if (p.splits == 1) {
        float inv;
        if (p.sink) {
            const float sk = p.sink[h], m2 = fmaxf(mf, sk), a2 = __expf(mf - m2);
            inv            = a2 / (lt * a2 + __expf(sk - m2));
        }
        else {
            inv = 1.f / lt;
        }
        inv *= ga_out_gate(p, t, h);
#pragma unroll
        for (int v = 0; v < VT; ++v) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int c = v * 16 + lg * 4 + r;
                if (c < V) {
                    ga_store<__bf16>(p, t, h, c, o[v][r] * inv);
                }
            }
        }
        return;
    }
    float* po = p.partial_o + (((size_t)t * p.q_heads + h) * p.splits + sp) * V;
    float* pm = p.partial_ml + (((size_t)t * p.q_heads + h) * p.splits + sp) * 2;
#pragma unroll
    for (int v = 0; v < VT; ++v) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int c = v * 16 + lg * 4 + r;
            if (c < V) {
                po[c] = o[v][r];
            }
        }
    }
    if (lg == 0) {
        pm[0] = mf;
        pm[1] = lt;
    }
}

bool general_attention_tiles_ok(const GeneralAttnParams& p)
{
    return p.elem_bytes == 2 && p.block_len == 64 && p.dim % 8 == 0 && p.vdim % 8 == 0 && p.dim <= 256 && p.vdim <= 256 && p.ldq % 8 == 0
           && p.cu_q && p.k_len && p.nseq >= 1 && p.max_q_len >= 1 && p.splits == 1 && p.q_heads % p.kv_heads == 0;
}

// row tiles per wave of the prefill kernel (64 * RT query rows per workgroup): as many as the register file holds without scratch --
// every key / value fragment a wave loads then serves 16 * RT query rows.  (Key sizes up to 256 with value sizes up to 192 -- the latent
// space of latent attention -- still hold two: 256 VGPRs + 184 AGPRs.)
constexpr int tile_rt(int ds, int vt)
{
    return (ds <= 4 && vt <= 8) ? 4 : ((ds <= 4 || vt <= 8 || (ds <= 8 && vt <= 12)) ? 2 : 1);
}

// value sizes are served by the next even tile count (the kernels test channel < vdim), key sizes by 1, 2, 3, 4, 6 or 8 steps
template<int DS>
static void launch_tiles_ds(const GeneralAttnParams& p, int arg, dim3 grid, hipStream_t st, bool decode)
{
    const int vt = (p.vdim + 15) / 16;
    switch (vt <= 1 ? 1 : (vt + 1) / 2 * 2) {
#define TM_TILE_CASE(VT_)                                                           \
    case VT_:                                                                       \
        if (decode) {                                                               \
            attn_decode_kernel<DS, VT_><<<grid, 256, 0, st>>>(p, arg);              \
        }                                                                           \
        else {                                                                      \
            attn_tiles_kernel<DS, VT_, tile_rt(DS, VT_)><<<grid, 256, 0, st>>>(p, arg); \
        }                                                                           \
        break;
        TM_TILE_CASE(1) TM_TILE_CASE(2) TM_TILE_CASE(4) TM_TILE_CASE(6) TM_TILE_CASE(8) TM_TILE_CASE(10) TM_TILE_CASE(12) TM_TILE_CASE(14)
        TM_TILE_CASE(16)
#undef TM_TILE_CASE
    }
}

static int launch_mfma(const GeneralAttnParams& p, int arg, dim3 grid, hipStream_t st, bool decode)
{
    const int ds = (p.dim + 31) / 32;
    switch (ds <= 4 ? ds : (ds <= 6 ? 6 : 8)) {
        case 1: launch_tiles_ds<1>(p, arg, grid, st, decode); break;
        case 2: launch_tiles_ds<2>(p, arg, grid, st, decode); break;
        case 3: launch_tiles_ds<3>(p, arg, grid, st, decode); break;
        case 4: launch_tiles_ds<4>(p, arg, grid, st, decode); break;
        case 6: launch_tiles_ds<6>(p, arg, grid, st, decode); break;
        default: launch_tiles_ds<8>(p, arg, grid, st, decode); break;
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

bool general_attention_decode_ok(const GeneralAttnParams& p)
{
    return p.elem_bytes == 2 && p.block_len == 64 && p.dim % 8 == 0 && p.vdim % 8 == 0 && p.dim <= 256 && p.vdim <= 256 && p.ldq % 8 == 0
           && p.q_heads % p.kv_heads == 0 && p.splits >= 1 && (p.splits == 1 || (p.partial_o && p.partial_ml));
}

int launch_general_attention_decode(const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(general_attention_decode_ok(p), "attention decode kernel: bf16, 64-token blocks, dim and vdim multiples of 8 up to 256");
    if (p.rows == 0) {
        return 0;
    }
    const int chunks = (p.q_heads / p.kv_heads + 15) / 16;
    TM_TRY_RC(launch_mfma(p, chunks, dim3(p.rows, p.kv_heads * chunks, p.splits), st, true));
    if (p.splits > 1) {
        launch_rows_merge<__bf16>(p, st);
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}

int launch_general_attention_tiles(const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(general_attention_tiles_ok(p), "attention tile kernel: bf16, 64-token blocks, dim and vdim multiples of 8 up to 256, sequence description");
    if (p.rows == 0) {
        return 0;
    }
    const int ds = (p.dim + 31) / 32, vt = (p.vdim + 15) / 16;
    const int rows = kTileRows * tile_rt(ds <= 4 ? ds : (ds <= 6 ? 6 : 8), vt <= 1 ? 1 : (vt + 1) / 2 * 2);  // the instantiation launch_mfma picks
    const int tiles_per_seq = (p.max_q_len + rows - 1) / rows;
    return launch_mfma(p, tiles_per_seq, dim3(p.nseq * tiles_per_seq, p.q_heads), st, false);
}

int launch_general_attention(const GeneralAttnParams& p, bool prefill, hipStream_t st)
{
    static const bool tiles_on = !getenv("TM_ATTN_TILES") || atoi(getenv("TM_ATTN_TILES")) != 0;  // A/B switch: 0 = row kernel everywhere
    if (prefill && tiles_on && general_attention_tiles_ok(p)) {
        return launch_general_attention_tiles(p, st);
    }
    if (!prefill && tiles_on && general_attention_decode_ok(p)) {
        return launch_general_attention_decode(p, st);
    }
    return launch_general_attention_rows(p, st);
}

}  // namespace tmk
