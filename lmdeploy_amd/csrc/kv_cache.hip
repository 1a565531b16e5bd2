// Paged KV cache: fused RoPE + online int8/int4 quantise-and-store, and dequantising flatten.
//
// Replaces: invokeProcessKV_v2_ / invokeFlattenKV_v2_ (src/turbomind/kernels/attention/kv_cache_utils_v2.cu
//           :18-210,340-468), the decode kernel's store prologue (attention_universal.h:273-330),
//           the quantiser (quantization.h:316-366,428-489) and FastRoPE (rotary_embedding.h:54-194).
//
// Integer contract (bit exact): per (token, kv head), K (after RoPE) and V separately
//   mn = min x, mx = max x; scale = h((f32(mx)-f32(mn)) * (1/(2^b-1))); zero = mn;
//   inv = h(1/f32(scale)); q = sat_u8(rne(h(h(x-zero)*inv))); b==4: min(q,15), nibbles [0,2,4,6,1,3,5,7].
// Byte layout of a block: kernels/attention/block.h:126-219 (KvLayout in tm_kernels.h).
//
// Work mapping: 16 lanes own one 128-wide head row (8 halves = 16 B each, coalesced 256 B per row);
// min/max are wave-level DPP reductions inside the 16-lane row -- no LDS.  HBM-bound byte work.
#include "tm_common.h"
#include "tm_kernels.h"

namespace tmk {

__device__ __forceinline__ int find_seq(const int* cu, int batch, int token)
{
    // largest b with cu[b] <= token   (cu has batch+1 entries, cu[0] = 0)
    int lo = 0, hi = batch;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (cu[mid] <= token) {
            lo = mid;
        }
        else {
            hi = mid;
        }
    }
    return lo;
}

__device__ __forceinline__ float row16_max(float v)
{
    v = fmaxf(v, dpp_f32<DPP_XOR1>(v));
    v = fmaxf(v, dpp_f32<DPP_XOR2>(v));
    v = fmaxf(v, dpp_f32<DPP_HMIRR>(v));
    v = fmaxf(v, dpp_f32<DPP_ROR8>(v));
    return v;
}

template<int BITS>
__global__ __launch_bounds__(256) void kv_rope_store_kernel(half_t* __restrict__ qkv,
                                                            int q_heads,
                                                            const int* __restrict__ cu_q_len,
                                                            const int* __restrict__ k_len,
                                                            int batch,
                                                            int total_tokens,
                                                            const half2_t* __restrict__ cos_sin,
                                                            int         max_pos,
                                                            KvCacheView cache)
{
    constexpr int  D       = 128;
    const KvLayout L       = cache.layout;
    const int      lane16  = threadIdx.x & 15;
    const int      token   = blockIdx.x * 16 + (threadIdx.x >> 4);
    const int      head    = blockIdx.y;  // [0,Hq): q   [Hq,Hq+Hkv): k   [Hq+Hkv, Hq+2Hkv): v
    const int      kv_heads = L.kv_heads;
    if (token >= total_tokens) {
        return;  // whole 16-lane rows exit together; DPP rows are 16 lanes
    }
    const int stride = (q_heads + 2 * kv_heads) * D;
    half_t*   src    = qkv + (size_t)token * stride + (size_t)head * D + lane16 * 8;
    half8_t   x      = *(const half8_t*)src;

    const int b       = find_seq(cu_q_len, batch, token);
    const int q_len   = cu_q_len[b + 1] - cu_q_len[b];
    const int history = k_len[b] - q_len;
    const int pos     = history + (token - cu_q_len[b]);

    const bool is_q = head < q_heads;
    const bool is_k = !is_q && head < q_heads + kv_heads;

    if ((is_q || is_k) && cos_sin != nullptr) {
        // interleaved pairs (x[2i], x[2i+1]); c,s already cast to fp16; fp16 mul/sub/add, no fma
        const int     p  = pos < max_pos ? pos : max_pos - 1;
        const half8_t cs = *(const half8_t*)(cos_sin + (size_t)p * (D / 2) + lane16 * 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const half_t c  = cs[2 * i];
            const half_t s  = cs[2 * i + 1];
            const half_t x0 = x[2 * i];
            const half_t x1 = x[2 * i + 1];
            const half_t a0 = c * x0;
            const half_t a1 = s * x1;
            const half_t b0 = c * x1;
            const half_t b1 = s * x0;
            x[2 * i]        = a0 - a1;
            x[2 * i + 1]    = b0 + b1;
        }
    }
    if (is_q) {
        *(half8_t*)src = x;
        return;
    }

    const int kv_head = is_k ? head - q_heads : head - q_heads - kv_heads;
    const int blk     = pos / L.block_len;
    const int ti      = pos - blk * L.block_len;
    char*     block   = (char*)cache.block_ptrs[cache.cu_block_nums[b] + blk] + cache.layer_offset;
    const int doff    = is_k ? L.k_data(kv_head, ti) : L.v_data(kv_head, ti);

    if constexpr (BITS == 16) {
        *(half8_t*)(block + doff + lane16 * 16) = x;
    }
    else {
        float mx = -INFINITY, mnn = -INFINITY;  // mnn tracks max(-x)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float f = (float)x[e];
            mx            = fmaxf(mx, f);
            mnn           = fmaxf(mnn, -f);
        }
        mx             = row16_max(mx);
        mnn            = row16_max(mnn);
        const float mn = -mnn;
        // fp16 min/max are exact in f32
        const float  inv_q_max = 1.0f / (float)((1 << BITS) - 1);
        const half_t scale     = (half_t)((mx - mn) * inv_q_max);
        const half_t zero      = (half_t)mn;
        const half_t inv       = (half_t)(1.0f / (float)scale);
        uint32_t     q[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const half_t d = x[e] - zero;
            const half_t y = d * inv;
            float        r = __builtin_rintf((float)y);  // RNE
            r              = (r == r) ? r : 0.0f;        // cvt.rni.sat of NaN -> 0
            r              = fminf(fmaxf(r, 0.0f), BITS == 8 ? 255.0f : 15.0f);
            q[e]           = (uint32_t)r;
        }
        if constexpr (BITS == 8) {
            u32x2 w;
            w[0] = q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24);
            w[1] = q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24);
            *(u32x2*)(block + doff + lane16 * 8) = w;
        }
        else {
            // nibble i of the word = element [0,2,4,6,1,3,5,7][i]   (quantization.h:459-471)
            const uint32_t w = q[0] | (q[2] << 4) | (q[4] << 8) | (q[6] << 12) | (q[1] << 16) | (q[3] << 20)
                               | (q[5] << 24) | (q[7] << 28);
            *(uint32_t*)(block + doff + lane16 * 4) = w;
        }
        if (lane16 == 0) {
            const int poff = is_k ? L.k_param(kv_head, ti) : L.v_param(kv_head, ti);
            half2_t   pr   = {scale, zero};
            *(half2_t*)(block + poff) = pr;
        }
    }
}

int launch_kv_rope_store(half_t*        qkv,
                         int            q_heads,
                         const int*     cu_q_len,
                         const int*     k_len,
                         int            batch,
                         int            total_tokens,
                         const half2_t* cos_sin,
                         int            max_pos,
                         KvCacheView    cache,
                         hipStream_t    st)
{
    TM_REQUIRE(cache.layout.head_dim == 128, "head_dim must be 128");
    TM_REQUIRE(cache.layout.bits == 16 || cache.layout.bits == 8 || cache.layout.bits == 4, "kv bits in {16,8,4}");
    if (total_tokens == 0) {
        return 0;
    }
    dim3 grid((total_tokens + 15) / 16, q_heads + 2 * cache.layout.kv_heads);
    switch (cache.layout.bits) {
        case 16:
            kv_rope_store_kernel<16><<<grid, 256, 0, st>>>(qkv, q_heads, cu_q_len, k_len, batch, total_tokens, cos_sin, max_pos, cache);
            break;
        case 8:
            kv_rope_store_kernel<8><<<grid, 256, 0, st>>>(qkv, q_heads, cu_q_len, k_len, batch, total_tokens, cos_sin, max_pos, cache);
            break;
        default:
            kv_rope_store_kernel<4><<<grid, 256, 0, st>>>(qkv, q_heads, cu_q_len, k_len, batch, total_tokens, cos_sin, max_pos, cache);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// ------------------------------------------------------------------------------------------------
// Flatten: one workgroup = 64 cached tokens (one block) of one (sequence, kv head).
//   K -> k_out[head][cu_k_off[b] + t][D];  V -> v_out[head][...][D] or transposed v_out[head][d][cu_k_off[b]+t]
// Dequant (two roundings, quantization.h:565-573,694-703): h(h(h(q)*scale) + zero).
// ------------------------------------------------------------------------------------------------
template<int BITS>
__device__ __forceinline__ half8_t load_dequant_flatten(const char* data, const char* param, int lane16)
{
    // returns dims [8*lane16, 8*lane16+8) of one token
    if constexpr (BITS == 16) {
        return *(const half8_t*)(data + lane16 * 16);
    }
    else {
        const half2_t pr = *(const half2_t*)param;
        const half_t  s = pr[0], z = pr[1];
        half8_t       o;
        if constexpr (BITS == 8) {
            const u32x2 w = *(const u32x2*)(data + lane16 * 8);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t qv = (w[e >> 2] >> (8 * (e & 3))) & 0xffu;
                const half_t   t  = (half_t)(float)qv * s;
                o[e]              = t + z;
            }
        }
        else {
            const uint32_t w = *(const uint32_t*)(data + lane16 * 4);
            constexpr int  nib_of[8] = {0, 4, 1, 5, 2, 6, 3, 7};  // element e sits in nibble nib_of[e]
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t qv = (w >> (4 * nib_of[e])) & 0xfu;
                const half_t   t  = (half_t)(float)qv * s;
                o[e]              = t + z;
            }
        }
        return o;
    }
}

template<int BITS, bool VT>
__global__ __launch_bounds__(256) void flatten_kv_kernel(half_t* __restrict__ k_out,
                                                         half_t* __restrict__ v_out,
                                                         const int* __restrict__ cu_k_off,
                                                         const int* __restrict__ k_len,
                                                         int         k_stride,
                                                         KvCacheView cache)
{
    constexpr int  D  = 128;
    const KvLayout L  = cache.layout;
    const int      b  = blockIdx.z;
    const int      hd = blockIdx.y;
    const int      t0 = blockIdx.x * 64;
    const int      n  = k_len[b];
    if (t0 >= n) {
        return;
    }
    __shared__ half_t vt_smem[VT ? 64 * (D + 8) : 1];

    const int    lane16 = threadIdx.x & 15;
    const int    row    = threadIdx.x >> 4;  // 16 token rows per pass
    const char*  block  = (const char*)cache.block_ptrs[cache.cu_block_nums[b] + blockIdx.x] + cache.layer_offset;
    const size_t obase  = (size_t)hd * k_stride + cu_k_off[b];

#pragma unroll
    for (int pass = 0; pass < 4; ++pass) {
        const int  ti    = pass * 16 + row;
        const bool valid = t0 + ti < n;
        half8_t    kk = {}, vv = {};
        if (valid) {
            kk = load_dequant_flatten<BITS>(block + L.k_data(hd, ti), block + L.k_param(hd, ti), lane16);
            vv = load_dequant_flatten<BITS>(block + L.v_data(hd, ti), block + L.v_param(hd, ti), lane16);
            *(half8_t*)(k_out + (obase + t0 + ti) * D + lane16 * 8) = kk;
            if constexpr (!VT) {
                *(half8_t*)(v_out + (obase + t0 + ti) * D + lane16 * 8) = vv;
            }
        }
        if constexpr (VT) {
            *(half8_t*)(vt_smem + ti * (D + 8) + lane16 * 8) = vv;  // zeros for invalid tokens
        }
    }
    if constexpr (VT) {
        __syncthreads();
        // thread -> (d = tid & 127, token octets); 64 tokens x 128 d = 1024 16-B vectors / 256 thr = 4 each
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int vec = threadIdx.x + it * 256;
            const int d   = vec & 127;
            const int to  = vec >> 7;  // 0..7 token octet
            half8_t   o;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                o[e] = vt_smem[(to * 8 + e) * (D + 8) + d];
            }
            // transposed layout: [head][d][k_stride]; padded tail tokens (>= n) are written as zeros,
            // the per-sequence region is 64-aligned by contract so this never spills into a neighbour
            *(half8_t*)(v_out + ((size_t)hd * D + d) * k_stride + cu_k_off[b] + t0 + to * 8) = o;
        }
    }
}

int launch_flatten_kv(half_t*     k_out,
                      half_t*     v_out,
                      int         transpose_v,
                      const int*  cu_k_off,
                      const int*  k_len,
                      int         batch,
                      int         max_k_len,
                      int         k_stride,
                      KvCacheView cache,
                      hipStream_t st)
{
    TM_REQUIRE(cache.layout.head_dim == 128, "head_dim must be 128");
    TM_REQUIRE(cache.layout.block_len == 64, "block_len must be 64");
    TM_REQUIRE(!transpose_v || k_stride % 64 == 0, "transposed V needs a 64-aligned k_stride");
    if (batch == 0 || max_k_len == 0) {
        return 0;
    }
    dim3 grid((max_k_len + 63) / 64, cache.layout.kv_heads, batch);
#define TM_FLATTEN(B_, T_) flatten_kv_kernel<B_, T_><<<grid, 256, 0, st>>>(k_out, v_out, cu_k_off, k_len, k_stride, cache)
    const int bits = cache.layout.bits;
    if (transpose_v) {
        if (bits == 16) TM_FLATTEN(16, true);
        else if (bits == 8) TM_FLATTEN(8, true);
        else TM_FLATTEN(4, true);
    }
    else {
        if (bits == 16) TM_FLATTEN(16, false);
        else if (bits == 8) TM_FLATTEN(8, false);
        else TM_FLATTEN(4, false);
    }
#undef TM_FLATTEN
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}


// ---- general layout: per layer and block, keys [kv_heads][block_len][dim] then values TRANSPOSED [kv_heads][vdim][block_len], bf16 | fp32:
// both are then K-contiguous operands of the attention kernels' matrix products (keys: channels run fastest; values: tokens run fastest) ------
__global__ void rows_prepare_kernel(int* __restrict__ row_seq, int* __restrict__ row_pos, const int* __restrict__ cu_q,
                                    const int* __restrict__ k_len, int nseq, int rows)
{
    const int t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= rows) {
        return;
    }
    const int base = cu_q[0];   // cu_q may count from an earlier row of the forward: row t here is row base + t there
    int lo = 0, hi = nseq - 1;  // the sequence with cu_q[s] <= base + t < cu_q[s + 1] (empty sequences are skipped by the search)
    while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (cu_q[mid] - base <= t) {
            lo = mid;
        }
        else {
            hi = mid - 1;
        }
    }
    row_seq[t] = lo;
    row_pos[t] = k_len[lo] - (cu_q[lo + 1] - cu_q[lo]) + (base + t - cu_q[lo]);
}

int launch_rows_prepare(int* row_seq, int* row_pos, const int* cu_q, const int* k_len, int nseq, int rows, hipStream_t st)
{
    TM_REQUIRE(row_seq && row_pos && cu_q && k_len && nseq >= 1, "rows_prepare: operands");
    if (rows > 0) {
        rows_prepare_kernel<<<(rows + 255) / 256, 256, 0, st>>>(row_seq, row_pos, cu_q, k_len, nseq, rows);
        TM_HIP_CHECK(hipGetLastError());
    }
    return 0;
}

template<class T>
__global__ void kv_store_general_kernel(const T* __restrict__ qkv, int ld, int k_col, int v_col, GeneralAttnParams p)
{
    const int kh = p.k_heads > 0 ? p.k_heads : p.kv_heads, vh = p.v_heads > 0 ? p.v_heads : p.kv_heads;
    const int per = kh * p.dim + vh * p.vdim;
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= (size_t)p.rows * per) {
        return;
    }
    const int t = (int)(i / per), c = (int)(i % per);
    const int s = p.row_seq[t], pos = p.row_pos[t];
    char* base = (char*)p.block_ptrs[(size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride + pos / p.block_len] + p.layer_offset;
    const int ti = pos % p.block_len;
    const int nk = kh * p.dim;
    if (c < nk) {
        const int g = c / p.dim, d = c % p.dim;
        ((T*)base)[((size_t)g * p.block_len + ti) * p.dim + d] = qkv[(size_t)t * ld + k_col + c];
    }
    else {
        const int cv = c - nk, g = cv / p.vdim, d = cv % p.vdim;
        ((T*)(base + p.v_offset))[((size_t)g * p.vdim + d) * p.block_len + ti] = qkv[(size_t)t * ld + v_col + cv];
    }
}

int launch_kv_store_general(const void* qkv, int ld, int k_col, int v_col, const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(qkv && p.row_seq && p.row_pos && p.block_ptrs && p.block_stride >= 1, "kv_store_general: operands");
    const int    kh = p.k_heads > 0 ? p.k_heads : p.kv_heads, vh = p.v_heads > 0 ? p.v_heads : p.kv_heads;
    const size_t n = (size_t)p.rows * (kh * p.dim + vh * p.vdim);
    if (n == 0) {
        return 0;
    }
    if (p.elem_bytes == 2) {
        kv_store_general_kernel<uint16_t><<<(n + 255) / 256, 256, 0, st>>>((const uint16_t*)qkv, ld, k_col, v_col, p);
    }
    else {
        kv_store_general_kernel<float><<<(n + 255) / 256, 256, 0, st>>>((const float*)qkv, ld, k_col, v_col, p);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// ---- projections of a mixer -> queries + paged cache, from the fp32 output of the fused projection GEMM ------------------------------
// Grouped-query attention whose queries, keys and values may each be scaled to unit root mean square per head (no weight): one wave per
// (row, head vector).  proj [rows][ld]: queries at q_col ([q_heads][dim]), keys at k_col ([kv_heads][dim]), values at v_col
// ([kv_heads][vdim]).  Queries go to q_out [rows][ldq] (head h at h * dim), keys / values into the cache in the general layout.
template<class T>
__global__ __launch_bounds__(256) void attn_prep_kernel(const float* __restrict__ proj, int ld, int q_col, int k_col, int v_col, T* __restrict__ q_out,
                                                        int ldq, int qk_norm, int v_norm, float eps, GeneralAttnParams p, AttnPrepExtra ex)
{
    const int lane = threadIdx.x & 63, t = blockIdx.x, u = blockIdx.y * 4 + (threadIdx.x >> 6);
    const int H = p.q_heads, G = p.k_heads > 0 ? p.k_heads : p.kv_heads, GV = p.v_heads > 0 ? p.v_heads : p.kv_heads;
    if (u >= H + G + GV) {
        return;
    }
    const int    kind = u < H ? 0 : (u < H + G ? 1 : 2), src = kind == 0 ? u : (kind == 1 ? u - H : u - H - G);
    const int    n    = kind == 2 ? p.vdim : p.dim;
    const int    col0 = (kind == 0 ? q_col : (kind == 1 ? k_col : v_col)) + src * n;
    const float* x    = proj + (size_t)t * ld + col0;
    __shared__ float conv_out[4][256];
    if (ex.conv_w) {  // one row per sequence: this wave owns the channels [col0, col0 + n) of the sequence's convolution state
        const int sq = p.row_seq[t], ps = p.row_pos[t], nh = ex.conv_taps - 1, C = ex.conv_ch;
        int       slot = p.seq_slot ? p.seq_slot[sq] : ex.conv_slot0 + sq;
        if (ex.conv_active && !ex.conv_active[sq]) {
            slot = ex.conv_park_slot;
        }
        float* st = ex.conv_state + (size_t)slot * ex.conv_slot_stride + ex.conv_offset;
        for (int i = lane; i < n; i += 64) {
            const int    ch = col0 + i;
            const float* w  = ex.conv_w + (size_t)ch * ex.conv_taps;
            const float  u  = x[i];
            float        acc = 0.f;
            for (int j = 0; j < nh; ++j) {
                acc = fmaf(w[j], ps > 0 ? st[(size_t)j * C + ch] : 0.f, acc);
            }
            acc = fmaf(w[nh], u, acc);
            for (int j = 0; j + 1 < nh; ++j) {
                st[(size_t)j * C + ch] = ps > 0 ? st[(size_t)(j + 1) * C + ch] : 0.f;
            }
            if (nh > 0) {
                st[(size_t)(nh - 1) * C + ch] = u;
            }
            conv_out[threadIdx.x >> 6][i] = acc;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        x = conv_out[threadIdx.x >> 6];
    }
    // several maps per head leave map-major: source [head][map] -> head map * (heads / maps) + head
    const int maps = kind == 2 ? 1 : ex.maps, cnt = kind == 0 ? H : G;
    const int head = maps > 1 ? (src % maps) * (cnt / maps) + src / maps : src;
    float     inv  = 1.f;
    if (kind == 2 ? v_norm : qk_norm) {
        float ss = 0.f;
        for (int i = lane; i < n; i += 64) {
            ss = fmaf(x[i], x[i], ss);
        }
        inv = 1.0f / sqrtf(group_sum<64>(ss) / (float)n + eps);
    }
    const int s = p.row_seq[t], pos = p.row_pos[t], ti = pos % p.block_len;
    // queries and keys: norm weight, then the rotation of the first rd channels (channel i pairs with i + rd / 2, or 2i with 2i + 1), all in fp32
    const float* nw = kind == 0 ? ex.q_w : (kind == 1 ? ex.k_w : nullptr);
    const int    rd = kind == 2 ? 0 : ex.rot_dims, half = rd / 2;
    auto         qk = [&](int i) {
        const float a = x[i] * inv * (nw ? nw[i] : 1.f);
        if (i >= rd) {
            return a;
        }
        const bool  first = ex.rot_pairs ? (i & 1) == 0 : i < half;
        const int   o = ex.rot_pairs ? (i ^ 1) : (i < half ? i + half : i - half);
        const float b = x[o] * inv * (nw ? nw[o] : 1.f);
        float       sn, cs;
        sincosf((float)pos * ex.inv_freq[ex.rot_pairs ? i >> 1 : (i < half ? i : i - half)], &sn, &cs);
        sn *= ex.rot_mult, cs *= ex.rot_mult;
        return first ? a * cs - b * sn : a * cs + b * sn;
    };
    if (kind == 0) {
        T* q = q_out + (size_t)t * ldq + (size_t)head * n;
        for (int i = lane; i < n; i += 64) {
            q[i] = (T)qk(i);
        }
        return;
    }
    char* base = (char*)p.block_ptrs[(size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride + pos / p.block_len] + p.layer_offset;
    if (kind == 1) {
        T* k = (T*)base + ((size_t)head * p.block_len + ti) * n;
        for (int i = lane; i < n; i += 64) {
            k[i] = (T)qk(i);
        }
    }
    else {
        T* v = (T*)(base + p.v_offset) + (size_t)head * n * p.block_len + ti;
        for (int i = lane; i < n; i += 64) {
            v[(size_t)i * p.block_len] = (T)(x[i] * inv);
        }
    }
}

int launch_attn_prep(const float* proj, int ld, int q_col, int k_col, int v_col, void* q_out, int ldq, bool qk_norm, bool v_norm, float eps,
                     const GeneralAttnParams& p, hipStream_t st, AttnPrepExtra ex)
{
    TM_REQUIRE(proj && q_out && p.row_seq && p.row_pos && p.block_ptrs && p.block_stride >= 1, "attn_prep: operands");
    TM_REQUIRE(ex.rot_dims >= 0 && ex.rot_dims % 2 == 0 && ex.rot_dims <= p.dim && (ex.rot_dims == 0 || ex.inv_freq), "attn_prep: rotation");
    const int kh = p.k_heads > 0 ? p.k_heads : p.kv_heads, vh = p.v_heads > 0 ? p.v_heads : p.kv_heads;
    TM_REQUIRE(ex.maps >= 1 && p.q_heads % ex.maps == 0 && kh % ex.maps == 0, "attn_prep: the maps divide the query and key heads");
    TM_REQUIRE(!ex.conv_w || (p.dim <= 256 && p.vdim <= 256 && ex.conv_taps >= 1 && ex.conv_ch >= 1 && (ex.conv_taps == 1 || ex.conv_state)),
               "attn_prep: fused convolution: head sizes up to 256, taps, channels, state");
    if (p.rows == 0) {
        return 0;
    }
    const dim3 grid(p.rows, (p.q_heads + kh + vh + 3) / 4);
    if (p.elem_bytes == 2) {
        attn_prep_kernel<__bf16><<<grid, 256, 0, st>>>(proj, ld, q_col, k_col, v_col, (__bf16*)q_out, ldq, qk_norm, v_norm, eps, p, ex);
    }
    else {
        attn_prep_kernel<float><<<grid, 256, 0, st>>>(proj, ld, q_col, k_col, v_col, (float*)q_out, ldq, qk_norm, v_norm, eps, p, ex);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// attention with mixed heads as attention over one wide key (see launch_talk_prep): grid (rows, head blocks) -- a workgroup forms the mixed
// queries of HB heads of one row (every workgroup computes the row's two norm statistics itself); head block 0 also writes the cache entry
template<class T>
__global__ __launch_bounds__(256) void talk_prep_kernel(const float* __restrict__ proj, int ld, int q_col, int k_col, T* __restrict__ q_out, int ldq,
                                                        const float* __restrict__ q_w, const float* __restrict__ k_w,
                                                        const float* __restrict__ talk, int D, int HB, float eps, GeneralAttnParams p)
{
    extern __shared__ float tp_lds[];  // the normed queries [H][D], then the mixing rows of this block's heads [HB][H]
    __shared__ float red[4];
    const int    t = blockIdx.x, H = p.q_heads, G = p.kv_heads, r = H / G, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int    h0 = blockIdx.y * HB, nh = min(HB, H - h0);
    float*       tk = tp_lds + H * D;
    const float *q = proj + (size_t)t * ld + q_col, *k = proj + (size_t)t * ld + k_col;
    auto block_sum = [&](float v) {
        v = group_sum<64>(v);
        __syncthreads();
        if (lane == 0) {
            red[wave] = v;
        }
        __syncthreads();
        return (red[0] + red[1]) + (red[2] + red[3]);
    };
    float sq = 0.f, sk = 0.f;
    for (int i = threadIdx.x; i < H * D; i += 256) {
        sq = fmaf(q[i], q[i], sq);
    }
    for (int i = threadIdx.x; i < G * D; i += 256) {
        sk = fmaf(k[i], k[i], sk);
    }
    const float qinv = 1.0f / sqrtf(block_sum(sq) / (float)(H * D) + eps);
    const float kinv = 1.0f / sqrtf(block_sum(sk) / (float)(G * D) + eps);
    for (int i = threadIdx.x; i < H * D; i += 256) {
        tp_lds[i] = q[i] * qinv * q_w[i];
    }
    for (int i = threadIdx.x; i < nh * H; i += 256) {
        tk[i] = talk[(size_t)h0 * H + i];
    }
    __syncthreads();
    // Q'[h][c D + d] = sum over the heads g of group c of talk[h][g] q_g[d]
    for (int i = threadIdx.x; i < nh * G * D; i += 256) {
        const int hl = i / (G * D), c = (i / D) % G, d = i % D;
        float     acc = 0.f;
        for (int g = c * r; g < (c + 1) * r; ++g) {
            acc = fmaf(tk[hl * H + g], tp_lds[g * D + d], acc);
        }
        q_out[(size_t)t * ldq + (size_t)h0 * G * D + i] = (T)acc;
    }
    if (blockIdx.y != 0) {
        return;
    }
    const int s = p.row_seq[t], pos = p.row_pos[t], ti = pos % p.block_len;
    char*     base = (char*)p.block_ptrs[(size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride + pos / p.block_len] + p.layer_offset;
    T*        kc   = (T*)base + (size_t)ti * (G * D);   // one key head of size G D
    T*        vc   = (T*)(base + p.v_offset) + ti;      // G value heads [D][block_len]: channel c D + d of the row at (c D + d) * block_len
    for (int i = threadIdx.x; i < G * D; i += 256) {
        kc[i]                         = (T)(k[i] * kinv * k_w[i]);
        vc[(size_t)i * p.block_len] = (T)k[i];
    }
}

int launch_talk_prep(const float* proj, int ld, int q_col, int k_col, void* q_out, int ldq, const float* q_w, const float* k_w, const float* talk,
                     int head_dim, float eps, const GeneralAttnParams& p, hipStream_t st)
{
    TM_REQUIRE(proj && q_out && q_w && k_w && talk && p.row_seq && p.row_pos && p.block_ptrs && p.block_stride >= 1, "talk_prep: operands");
    TM_REQUIRE(head_dim >= 1 && p.kv_heads >= 1 && p.q_heads % p.kv_heads == 0 && p.k_heads == 1 && p.v_heads == p.kv_heads
                   && p.dim == p.kv_heads * head_dim && p.vdim == head_dim && ldq >= p.q_heads * p.dim,
               "talk_prep: one key head of kv_heads * head_dim channels, kv_heads value heads of head_dim");
    TM_REQUIRE((size_t)p.q_heads * head_dim * 4 <= 48 * 1024, "talk_prep: heads * dim <= 12288");
    if (p.rows == 0) {
        return 0;
    }
    // few rows (decoded tokens): one head per workgroup so that the launch still fills the device; many rows: as few head blocks as keep
    // the mixing rows in LDS, the norm statistics are then computed once per row
    const int H = p.q_heads;
    int       hb = p.rows >= 512 ? H : std::max(1, (int)((int64_t)H * p.rows / 512));
    hb           = std::min(hb, std::max(1, (15 * 1024 - H * head_dim) / H));
    const size_t lds = ((size_t)H * head_dim + (size_t)hb * H) * 4;
    const dim3   grid(p.rows, (H + hb - 1) / hb);
    if (p.elem_bytes == 2) {
        talk_prep_kernel<__bf16><<<grid, 256, lds, st>>>(proj, ld, q_col, k_col, (__bf16*)q_out, ldq, q_w, k_w, talk, head_dim, hb, eps, p);
    }
    else {
        talk_prep_kernel<float><<<grid, 256, lds, st>>>(proj, ld, q_col, k_col, (float*)q_out, ldq, q_w, k_w, talk, head_dim, hb, eps, p);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// Latent attention: per token ONE normed latent vector c (size C) and ONE rotated key part (size R) shared by all heads are cached; a
// head's keys and values are linear images of c.  The cache entry is the key [c | rotated part] (p.dim = C + R, one key head) and the
// value c (p.vdim = C): attention then runs in the latent space -- the query's unrotated part is carried through the key expansion
// beforehand (q_plain . (U c) = (U^T q_plain) . c), the value expansion is applied to the attention output.
// proj [rows][ld]: queries at q_col, head h as [D unrotated | R rotated]; at dkv_col the C latent channels, then the R rotated ones.
//   q_plain [rows][ldp], head h at h * plain_stride : unrotated query parts (input of the key-expansion product)
//   q_full  [rows][ldq], head h at h * (C + R)      : the rotated part goes to [C, C + R) (the product fills [0, C))
// Rotation turns the first `rd` of the R channels: channel i pairs with i + rd / 2, angle = position * inv_freq[i], fp32; the rest pass.
template<class T>
__global__ __launch_bounds__(256) void latent_prep_kernel(const float* __restrict__ proj, int ld, int q_col, int dkv_col, T* __restrict__ q_plain,
                                                          int ldp, int plain_stride, T* __restrict__ q_full, int ldq,
                                                          const float* __restrict__ c_norm_w, const float* __restrict__ inv_freq, int D, int R, int C,
                                                          int rd, float eps, GeneralAttnParams p)
{
    __shared__ float red[4];
    const int    t = blockIdx.x, H = p.q_heads, half = rd / 2, still = R - rd;
    const int    s = p.row_seq[t], pos = p.row_pos[t], ti = pos % p.block_len;
    const float* x = proj + (size_t)t * ld;
    for (int i = threadIdx.x; i < H * D; i += 256) {
        const int h = i / D, d = i % D;
        q_plain[(size_t)t * ldp + (size_t)h * plain_stride + d] = (T)x[q_col + h * (D + R) + d];
    }
    for (int i = threadIdx.x; i < H * half; i += 256) {
        const int   h = i / half, f = i % half;
        const float u = x[q_col + h * (D + R) + D + f], v = x[q_col + h * (D + R) + D + f + half];
        float       sn, cs;
        sincosf((float)pos * inv_freq[f], &sn, &cs);
        T* q = q_full + (size_t)t * ldq + (size_t)h * (C + R) + C;
        q[f]        = (T)(u * cs - v * sn);
        q[f + half] = (T)(v * cs + u * sn);
    }
    for (int i = threadIdx.x; i < H * still; i += 256) {  // channels of the rotated part that do not turn
        const int h = i / still, f = rd + i % still;
        q_full[(size_t)t * ldq + (size_t)h * (C + R) + C + f] = (T)x[q_col + h * (D + R) + D + f];
    }
    char* base = (char*)p.block_ptrs[(size_t)(p.seq_slot ? p.seq_slot[s] : s) * p.block_stride + pos / p.block_len] + p.layer_offset;
    T*    k    = (T*)base + (size_t)ti * (C + R);
    T*    vt   = (T*)(base + p.v_offset) + ti;
    float ss   = 0.f;
    for (int i = threadIdx.x; i < C; i += 256) {
        ss = fmaf(x[dkv_col + i], x[dkv_col + i], ss);
    }
    ss = group_sum<64>(ss);
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = ss;
    }
    __syncthreads();
    const float inv = 1.0f / sqrtf(((red[0] + red[1]) + (red[2] + red[3])) / (float)C + eps);
    for (int i = threadIdx.x; i < C; i += 256) {
        const T c = (T)(x[dkv_col + i] * inv * c_norm_w[i]);
        k[i]                          = c;
        vt[(size_t)i * p.block_len] = c;
    }
    for (int f = threadIdx.x; f < half; f += 256) {
        const float u = x[dkv_col + C + f], v = x[dkv_col + C + f + half];
        float       sn, cs;
        sincosf((float)pos * inv_freq[f], &sn, &cs);
        k[C + f]        = (T)(u * cs - v * sn);
        k[C + f + half] = (T)(v * cs + u * sn);
    }
    for (int f = rd + threadIdx.x; f < R; f += 256) {
        k[C + f] = (T)x[dkv_col + C + f];
    }
}

int launch_latent_prep(const float* proj, int ld, int q_col, int dkv_col, void* q_plain, int ldp, int plain_stride, void* q_full, int ldq,
                       const float* c_norm_w, const float* inv_freq, int D, int R, int C, int rd, float eps, const GeneralAttnParams& p,
                       hipStream_t st)
{
    TM_REQUIRE(proj && q_plain && q_full && c_norm_w && inv_freq && p.row_seq && p.row_pos && p.block_ptrs, "latent_prep: operands");
    TM_REQUIRE(rd % 2 == 0 && rd >= 0 && rd <= R && p.kv_heads == 1 && p.dim == C + R && p.vdim == C && plain_stride >= D, "latent_prep: sizes");
    if (p.rows == 0) {
        return 0;
    }
    if (p.elem_bytes == 2) {
        latent_prep_kernel<__bf16><<<p.rows, 256, 0, st>>>(proj, ld, q_col, dkv_col, (__bf16*)q_plain, ldp, plain_stride, (__bf16*)q_full, ldq, c_norm_w,
                                                           inv_freq, D, R, C, rd, eps, p);
    }
    else {
        latent_prep_kernel<float><<<p.rows, 256, 0, st>>>(proj, ld, q_col, dkv_col, (float*)q_plain, ldp, plain_stride, (float*)q_full, ldq, c_norm_w,
                                                          inv_freq, D, R, C, rd, eps, p);
    }
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

}  // namespace tmk
