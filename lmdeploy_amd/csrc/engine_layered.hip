// Layer-list model family on the engine: a decoder given as a list of residual blocks (tm_layered_config), each with its mixer, the
// mixer's sizes and constants and its feed-forward.  Everything around the layer loop is the engine's own: block pool and block tables,
// the batch description of forward() (decode / prefill / mixed), the scheduler, sampling, graph capture of the decode step.
//
// Per layer (weights of layer `src`, cache of the layer itself):
//   h1, h2   = norm1(x), norm2(x)                    one launch, one statistic (launch_rmsnorm_f32)
//   [q|k|v]  = h1 . Wqkv^T                           one GEMM over the concatenated projections
//   K, V    -> paged cache; attention -> cat[:, 0 : heads * vdim]
//   cat[:, heads * vdim :] = act(h2 . Wup^T)         activation in the GEMM epilogue
//   x       += residual_mult * (cat . [Wo | Wdown]^T)   ONE GEMM over the concatenated inputs closes the block in its epilogue
// The residual stream x is fp32; h, q, k, v, cat and the cache are bf16 (TM_DTYPE_BF16) or fp32 (TM_DTYPE_F32).
//
// "Wide" blocks (LmLayer::wide: per-head norms, rotation, gates or routers read the projections in fp32) run
//   x        = loop.in [x | x0] + loop.step[t]          only where a loop pass begins (concat + GEMM with a bias epilogue)
//   h        = norm1(x)
//   proj     = h . [q | k | v | gates | router]^T       ONE GEMM, fp32 output
//   queries, cache  <- proj                             launch_attn_prep (unit norms) | launch_latent_prep (norm, rotation)
//   latent:  q[:, head, 0:C] = q_plain[:, head] . uk_head          one batched GEMM (the key expansion carried to the query)
//   attention (chunk, distance penalty, sink, output gate as parameters)
//   latent:  cat[:, head] = lat[:, head] . uv_head^T               one batched GEMM (the value expansion)
//   x       += sigmoid(proj[rg1] + b1) * (cat . Wo^T)              GEMM with the gated-residual epilogue
//   dense:   a = act(h . gate^T) * (h . up^T)  ONE GEMM over the interleaved [gate | up] image, activation in its epilogue;
//            x += sigmoid(proj[rg2] + b2) * (a . Wdown^T)
//   experts: router top-k -> rows sorted by expert, scaled by their score -> the same two products batched over the experts -> gated sum
//
// Post-norm blocks (LmLayer::post): the sublayers read the stream itself and a layer norm with bias follows them,
//   h        = x in the activation type                  (written by the previous block's closing launch)
//   proj     = h . [every projection of the mixer]^T + bias       ONE GEMM, fp32 output
//   attention:  launch_attn_prep (weighted per-head norms, rotation) -> paged cache; attention with a window + kept first tokens
//   lightning / delta rule:  launch_state_mix on the slot's recurrent state (fp32) -> gated group norm
//   y        = cat . Wo^T (fp32);   x += LN1(y), h = x            one launch
//   dense:   y = down(xielu(up h));   experts: soft-max router top-k -> rows sorted by expert -> two batched products -> weighted sum
//            (+ the shared expert);   x += LN2(y), h = x
//
// Post-norm blocks with RMS group norms (spec.norm_groups > 0; group_layer()): x += GN1(mixer(x)); x += GN2(ff(x)),
//   proj     = h . [every projection of the mixer]^T               ONE GEMM, fp32 output
//   conv     = short causal convolution of the q, k, v columns (its last inputs live in the slot's state)      launch_short_conv
//   differential attention:  launch_attn_prep (two maps per head leave as heads of their own; norm, pairwise rotation) -> attention over
//            2 G key heads and G value heads, fp32 output -> o = a1 - lambda a2, unit RMS per head (launch_diff_head_norm) -> Wo
//   parallel: left  = launch_talk_prep (norms over the whole projection; the head-mixing matrix folded into the queries) -> attention over
//                     one wide key with a distance table and a zero sink -> sigmoid gate -> Wo (left)
//             right = conv + silu -> decay / gate inner products -> launch_gdelta_prep -> launch_state_mix -> gated head norm -> Wo (right)
//             x += GN1(0.5 (rms(left) w_l + rms(right) w_r)), h = x                                              one launch
//   gated feed-forward: act(gate h) * (up h) in the epilogue of ONE product, down; x += GN2(y), h = x
#include "engine_internal.h"

namespace tmk {

// out[0] = softplus(p), out[1] = 1/2 + softplus(q): the two numbers of the xIELU activation as the GEMM epilogue reads them
__global__ void xielu_par_kernel(float* out, const uint16_t* in)
{
    if (threadIdx.x < 2) {
        const float v      = __builtin_bit_cast(float, (uint32_t)in[threadIdx.x] << 16);
        const float sp     = v > 20.f ? v : log1pf(expf(v));
        out[threadIdx.x] = threadIdx.x == 0 ? sp : 0.5f + sp;
    }
}

__global__ void fill_normal_bf16_kernel(uint16_t* out, size_t n, float mean, float stddev, uint64_t seed)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    uint64_t z = (i + 1) * 0x9E3779B97F4A7C15ull + seed * 0xD1B54A32D192ED03ull;
    z          = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z          = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    const float u1 = ((float)(uint32_t)(z >> 40) + 1.0f) * (1.0f / 16777217.0f);
    const float u2 = (float)(uint32_t)((z >> 8) & 0xffffffu) * (1.0f / 16777216.0f);
    const float v  = mean + stddev * sqrtf(-2.0f * __logf(u1)) * __cosf(6.283185307179586f * u2);
    const __bf16 b = (__bf16)v;
    out[i]         = __builtin_bit_cast(uint16_t, b);
}

// checkpoint bf16 vector -> fp32 (norm weights, sinks)
__global__ void bf16_to_f32_kernel(float* out, const uint16_t* in, size_t n)
{
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        out[i] = __builtin_bit_cast(float, (uint32_t)in[i] << 16);
    }
}

// lambda of differential attention: exp(lq1 . lk1) - exp(lq2 . lk2) + init, from the checkpoint's bf16 vectors
__global__ void diff_lambda_kernel(float* out, const uint16_t* q1, const uint16_t* k1, const uint16_t* q2, const uint16_t* k2, int n, float init)
{
    auto f = [](uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); };
    float a = 0.f, b = 0.f;
    for (int i = threadIdx.x; i < n; i += 64) {
        a = fmaf(f(q1[i]), f(k1[i]), a);
        b = fmaf(f(q2[i]), f(k2[i]), b);
    }
    a = group_sum<64>(a), b = group_sum<64>(b);
    if (threadIdx.x == 0) {
        out[0] = expf(a) - expf(b) + init;
    }
}

__global__ void iota_kernel(int* out, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        out[i] = i;
    }
}

static_assert(kActRelu2 == TM_ACT_RELU2 && kActGeluTanh == TM_ACT_GELU_TANH && kActSilu == TM_ACT_SILU, "activation codes");

static std::string lname(int i, const char* t)
{
    return "l" + std::to_string(i) + "." + t;
}

// blocks whose projections are read in fp32 before they become queries, cache entries, gates or router scores
static bool layer_wide(const tm_layer_spec& s)
{
    return s.mixer == TM_MIXER_LATENT || s.one_norm || s.resid_gate || s.qk_unit_norm || s.v_unit_norm || s.out_gate || s.mlp == TM_MLP_GATED
           || s.mlp == TM_MLP_MOE;
}

static int to_f32(tm_engine* e, const std::string& name, size_t n, float** out)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled, "weight not loaded: " + name);
    TM_TRY(dmalloc(out, n));
    bf16_to_f32_kernel<<<(n + 255) / 256, 256, 0, e->stream>>>(*out, (const uint16_t*)s.dev, n);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

static int place(tm_engine* e, DenseWeight& d, int row0, int col0, const std::string& name, int rows, int cols, size_t src_row = 0, int item = 0,
                 bool transpose = false, int half = 0)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled, "weight not loaded: " + name);
    TM_REQUIRE((int64_t)(src_row + rows) * cols * 2 <= s.bytes, "internal: weight part outside " + name);
    return dense_weight_place(d, row0, col0, (const uint16_t*)s.dev + src_row * cols, rows, cols, e->stream, item, transpose, half);
}

static int process_wide_layer(tm_engine* e, int i, LmLayer& L, int dt)
{
    const tm_layer_spec& s = L.spec;
    const int            W = e->lm->cfg.width, H = s.heads;
    TM_TRY(dense_weight_alloc(L.qkv, W, L.c_router + (s.mlp == TM_MLP_MOE ? s.experts : 0), dt, e->stream));
    TM_TRY(place(e, L.qkv, 0, 0, lname(i, "mix.q"), L.n_q, W));
    if (s.mixer == TM_MIXER_LATENT) {
        const int C = s.kv_rank, R = s.rot_dim;
        TM_TRY(place(e, L.qkv, L.c_k, 0, lname(i, "mix.dkv"), C + R, W));
        TM_TRY(to_f32(e, lname(i, "mix.dkv.norm"), C, &L.c_norm));
        TM_TRY(dense_weight_alloc(L.uk, s.dim, C, dt, e->stream, H));
        TM_TRY(dense_weight_alloc(L.uv, C, s.vdim, dt, e->stream, H));
        for (int h = 0; h < H; ++h) {  // uk rows [h dim, (h + 1) dim) are head h's [dim][kv_rank]: stored transposed, kv_rank outputs of dim inputs
            TM_TRY(place(e, L.uk, 0, 0, lname(i, "mix.uk"), s.dim, C, (size_t)h * s.dim, h, true));
            TM_TRY(place(e, L.uv, 0, 0, lname(i, "mix.uv"), s.vdim, C, (size_t)h * s.vdim, h, false));
        }
        const int          rd = s.rot_dims > 0 ? s.rot_dims : R;
        std::vector<float> f(rd / 2);
        for (int j = 0; j < rd / 2; ++j) {
            f[j] = (float)std::pow((double)s.rot_base, -2.0 * j / rd);
        }
        TM_TRY(dmalloc(&L.inv_freq, (size_t)std::max(1, rd / 2)));
        if (!f.empty()) {
            TM_HIP_CHECK(hipMemcpyAsync(L.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice, e->stream));
        }
        TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    }
    else {
        TM_TRY(place(e, L.qkv, L.c_k, 0, lname(i, "mix.k"), L.a_kv * s.dim, W));
        TM_TRY(place(e, L.qkv, L.c_v, 0, lname(i, "mix.v"), L.a_kv * s.vdim, W));
        if (s.out_gate) {
            TM_TRY(place(e, L.qkv, L.c_g, 0, lname(i, "mix.g"), H, W));
        }
    }
    if (s.dist_bias) {
        TM_TRY(to_f32(e, lname(i, "mix.r1"), H, &L.r1));
        TM_TRY(to_f32(e, lname(i, "mix.r2"), H, &L.r2));
    }
    if (s.sink) {
        TM_TRY(to_f32(e, lname(i, "mix.sink"), H, &L.sink));
    }
    TM_TRY(to_f32(e, lname(i, "norm1"), W, &L.norm1));
    TM_TRY(dense_weight_alloc(L.wo, L.n_att, W, dt, e->stream));
    TM_TRY(place(e, L.wo, 0, 0, lname(i, "mix.o"), W, L.n_att));
    if (s.resid_gate) {
        TM_TRY(place(e, L.qkv, L.c_rg1, 0, lname(i, "rg1"), W, W));
        TM_TRY(to_f32(e, lname(i, "rg1.b"), W, &L.rg1_b));
        if (s.mlp) {
            TM_TRY(place(e, L.qkv, L.c_rg2, 0, lname(i, "rg2"), W, W));
            TM_TRY(to_f32(e, lname(i, "rg2.b"), W, &L.rg2_b));
        }
    }
    if (s.mlp == TM_MLP_GATED) {
        TM_TRY(dense_weight_alloc(L.gu, W, dense_pair_rows(s.ff), dt, e->stream));  // gate and up interleaved: the activation is the GEMM's epilogue
        TM_TRY(place(e, L.gu, 0, 0, lname(i, "mlp.gate"), s.ff, W, 0, 0, false, 1));
        TM_TRY(place(e, L.gu, 0, 0, lname(i, "mlp.up"), s.ff, W, 0, 0, false, 2));
        TM_TRY(dense_weight_alloc(L.down, s.ff, W, dt, e->stream));
        TM_TRY(place(e, L.down, 0, 0, lname(i, "mlp.down"), W, s.ff));
    }
    else if (s.mlp == TM_MLP_MOE) {
        TM_TRY(place(e, L.qkv, L.c_router, 0, lname(i, "mlp.router"), s.experts, W));
        TM_TRY(dense_weight_alloc(L.gu, W, dense_pair_rows(s.ff), dt, e->stream, s.experts));
        TM_TRY(dense_weight_alloc(L.down, s.ff, W, dt, e->stream, s.experts));
        for (int x = 0; x < s.experts; ++x) {
            const std::string ex = "mlp.e" + std::to_string(x) + ".";
            TM_TRY(place(e, L.gu, 0, 0, lname(i, (ex + "gate").c_str()), s.ff, W, 0, x, false, 1));
            TM_TRY(place(e, L.gu, 0, 0, lname(i, (ex + "up").c_str()), s.ff, W, 0, x, false, 2));
            TM_TRY(place(e, L.down, 0, 0, lname(i, (ex + "down").c_str()), W, s.ff, 0, x));
        }
    }
    return 0;
}

// bf16 vector of a slot -> fp32 at out[0 .. n)
static int to_f32_at(tm_engine* e, const std::string& name, size_t n, float* out)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled, "weight not loaded: " + name);
    bf16_to_f32_kernel<<<(n + 255) / 256, 256, 0, e->stream>>>(out, (const uint16_t*)s.dev, n);
    TM_HIP_CHECK(hipGetLastError());
    return 0;
}

// a bf16 vector / matrix of a slot on the host, as floats
static int slot_to_host(tm_engine* e, const std::string& name, size_t n, std::vector<float>& out)
{
    Slot& s = e->slots[name];
    TM_REQUIRE(s.filled && (int64_t)n * 2 <= s.bytes, "weight not loaded: " + name);
    std::vector<uint16_t> raw(n);
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    TM_HIP_CHECK(hipMemcpy(raw.data(), s.dev, n * 2, hipMemcpyDeviceToHost));
    out.resize(n);
    for (size_t i = 0; i < n; ++i) {
        const uint32_t b = (uint32_t)raw[i] << 16;
        memcpy(&out[i], &b, 4);
    }
    return 0;
}

static int upload_f32(tm_engine* e, const std::vector<float>& v, float** out)
{
    TM_TRY(dmalloc(out, std::max<size_t>(1, v.size())));
    if (!v.empty()) {
        TM_HIP_CHECK(hipMemcpy(*out, v.data(), v.size() * 4, hipMemcpyHostToDevice));
    }
    return 0;
}

// rotation frequencies of the first `dims` channels of a head; yarn_factor > 0: the slow frequencies are divided by it, with a linear ramp
// between the channel that turns `fast` times over `original` positions and the one that turns `slow` times (see tm_layer_spec)
static std::vector<float> rotation_frequencies(const tm_layer_spec& s)
{
    const int          dims = s.rot_dims;
    std::vector<float> f(dims / 2);
    const double       base = s.rot_base;
    double             lo = 0, hi = 0;
    if (s.yarn_factor > 0.f) {
        auto dim_of = [&](double turns) { return dims * std::log((double)s.yarn_original / (2.0 * M_PI * turns)) / (2.0 * std::log(base)); };
        lo = std::max(std::floor(dim_of(s.yarn_fast)), 0.0);
        hi = std::min(std::ceil(dim_of(s.yarn_slow)), (double)dims - 1.0);
    }
    for (int j = 0; j < dims / 2; ++j) {
        double v = std::pow(base, -2.0 * j / dims) / (double)s.rot_scale;
        if (s.yarn_factor > 0.f) {
            const double ramp = std::min(1.0, std::max(0.0, (j - lo) / std::max(hi - lo, 0.001)));
            v                 = v / (double)s.yarn_factor * ramp + v * (1.0 - ramp);
        }
        f[j] = (float)v;
    }
    return f;
}

// post-norm blocks with RMS group norms: differential attention with convolved projections, or the parallel pair (see the head of this file)
static int process_group_layer(tm_engine* e, int i, LmLayer& L, int dt)
{
    const tm_layer_spec& s = L.spec;
    const int            W = e->lm->cfg.width, H = s.heads;
    hipStream_t          st = e->stream;
    TM_TRY(dense_weight_alloc(L.qkv, W, L.c_end, dt, st));
    auto conv_weights = [&](const char* pre, int nq, int nk, int nv, int taps) -> int {
        TM_TRY(dmalloc(&L.conv_w, (size_t)(nq + nk + nv) * taps));
        TM_TRY(to_f32_at(e, lname(i, (std::string(pre) + "q.conv").c_str()), (size_t)nq * taps, L.conv_w));
        TM_TRY(to_f32_at(e, lname(i, (std::string(pre) + "k.conv").c_str()), (size_t)nk * taps, L.conv_w + (size_t)nq * taps));
        TM_TRY(to_f32_at(e, lname(i, (std::string(pre) + "v.conv").c_str()), (size_t)nv * taps, L.conv_w + (size_t)(nq + nk) * taps));
        return 0;
    };
    if (s.mixer == TM_MIXER_ATTENTION) {
        TM_TRY(place(e, L.qkv, 0, 0, lname(i, "mix.q"), L.n_q, W));
        TM_TRY(place(e, L.qkv, L.c_k, 0, lname(i, "mix.k"), L.n_k, W));
        TM_TRY(place(e, L.qkv, L.c_v, 0, lname(i, "mix.v"), L.n_v, W));
        if (s.qk_norm_w) {
            TM_TRY(to_f32(e, lname(i, "mix.q.norm"), s.dim, &L.q_w));
            TM_TRY(to_f32(e, lname(i, "mix.k.norm"), s.dim, &L.k_w));
        }
        if (s.rot_dims > 0) {
            TM_TRY(upload_f32(e, rotation_frequencies(s), &L.inv_freq));
        }
        if (s.conv_taps > 0) {
            TM_TRY(conv_weights("mix.", L.n_q, L.n_k, L.n_v, s.conv_taps));
        }
        if (s.diff_maps) {
            TM_TRY(dmalloc(&L.lambda, (size_t)1));
            const char* names[4] = {"mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"};
            const uint16_t* v[4];
            for (int j = 0; j < 4; ++j) {
                Slot& sl = e->slots[lname(i, names[j])];
                TM_REQUIRE(sl.filled, "weight not loaded: " + lname(i, names[j]));
                v[j] = (const uint16_t*)sl.dev;
            }
            diff_lambda_kernel<<<1, 64, 0, st>>>(L.lambda, v[0], v[1], v[2], v[3], s.dim, s.diff_init);
            TM_HIP_CHECK(hipGetLastError());
        }
        TM_TRY(dense_weight_alloc(L.wo, L.n_att, W, dt, st));
        TM_TRY(place(e, L.wo, 0, 0, lname(i, "mix.o"), W, L.n_att));
    }
    else {  // parallel: [left q | left k | left gate | right q | right k | right v | beta | a1 | g1]
        const int Hr = s.r_heads, dr = s.r_dim, dvr = s.r_vdim;
        TM_TRY(place(e, L.qkv, 0, 0, lname(i, "mix.left.q"), L.n_q, W));
        TM_TRY(place(e, L.qkv, L.c_k, 0, lname(i, "mix.left.k"), L.n_k, W));
        TM_TRY(place(e, L.qkv, L.c_g, 0, lname(i, "mix.left.g"), L.n_att, W));
        TM_TRY(place(e, L.qkv, L.c_rq, 0, lname(i, "mix.right.q"), L.r_nqk, W));
        TM_TRY(place(e, L.qkv, L.c_rk, 0, lname(i, "mix.right.k"), L.r_nqk, W));
        TM_TRY(place(e, L.qkv, L.c_rv, 0, lname(i, "mix.right.v"), L.r_nv, W));
        TM_TRY(place(e, L.qkv, L.c_b, 0, lname(i, "mix.right.b"), Hr, W));
        TM_TRY(place(e, L.qkv, L.c_a1, 0, lname(i, "mix.right.a1"), s.a_rank, W));
        TM_TRY(place(e, L.qkv, L.c_g1, 0, lname(i, "mix.right.g1"), s.g_rank, W));
        TM_TRY(to_f32(e, lname(i, "mix.left.q.norm"), L.n_q, &L.q_w));
        TM_TRY(to_f32(e, lname(i, "mix.left.k.norm"), L.n_k, &L.k_w));
        TM_TRY(to_f32(e, lname(i, "mix.left.talk"), (size_t)H * H, &L.talk));
        {   // the distance bias after the head mixing, per head and distance: tab[h][d] = sum_g talk[h][g] rel[bucket(d)][g]
            std::vector<float> rel, talk;
            const int          B = s.dist_buckets, half = B / 2;
            TM_TRY(slot_to_host(e, lname(i, "mix.left.rel"), (size_t)B * H, rel));
            TM_TRY(slot_to_host(e, lname(i, "mix.left.talk"), (size_t)H * H, talk));
            L.dist_len = s.window > 0 ? std::min(s.window, e->cfg.session_len) : e->cfg.session_len;
            std::vector<float> tab((size_t)H * L.dist_len);
            const double       span = std::log((double)s.dist_max / std::max(half, 1));
            for (int d = 0; d < L.dist_len; ++d) {
                int b = d;
                if (d >= half) {
                    b = half > 0 ? std::min(B - 1, half + (int)std::floor(std::log((double)d / half) / span * (B - half))) : B - 1;
                }
                for (int h = 0; h < H; ++h) {
                    double acc = 0;
                    for (int g = 0; g < H; ++g) {
                        acc += (double)talk[(size_t)h * H + g] * (double)rel[(size_t)b * H + g];
                    }
                    tab[(size_t)h * L.dist_len + d] = (float)acc;
                }
            }
            TM_TRY(upload_f32(e, tab, &L.dist_tab));
        }
        TM_TRY(upload_f32(e, std::vector<float>(H, 0.f), &L.zero_sink));
        TM_TRY(dense_weight_alloc(L.wo, L.n_att, W, dt, st));
        TM_TRY(place(e, L.wo, 0, 0, lname(i, "mix.left.o"), W, L.n_att));
        TM_TRY(dense_weight_alloc(L.wo_r, L.r_nv, W, dt, st));
        TM_TRY(place(e, L.wo_r, 0, 0, lname(i, "mix.right.o"), W, L.r_nv));
        TM_TRY(dense_weight_alloc(L.a2, s.a_rank, Hr * dr, dt, st));
        TM_TRY(place(e, L.a2, 0, 0, lname(i, "mix.right.a2"), Hr * dr, s.a_rank));
        TM_TRY(dense_weight_alloc(L.g2, s.g_rank, L.r_nv, dt, st));
        TM_TRY(place(e, L.g2, 0, 0, lname(i, "mix.right.g2"), L.r_nv, s.g_rank));
        TM_TRY(to_f32(e, lname(i, "mix.right.A_log"), Hr, &L.a_log));
        TM_TRY(to_f32(e, lname(i, "mix.right.dt_bias"), (size_t)Hr * dr, &L.dt_bias));
        {   // the head norm's weight [vdim] is shared by the heads: one copy per head for the gated head norm
            std::vector<float> nw, all;
            TM_TRY(slot_to_host(e, lname(i, "mix.right.norm"), dvr, nw));
            for (int h = 0; h < Hr; ++h) {
                all.insert(all.end(), nw.begin(), nw.end());
            }
            TM_TRY(upload_f32(e, all, &L.r_norm));
        }
        TM_TRY(conv_weights("mix.right.", L.r_nqk, L.r_nqk, L.r_nv, s.r_conv));
        TM_TRY(to_f32(e, lname(i, "mix.left.out"), W, &L.join_l));
        TM_TRY(to_f32(e, lname(i, "mix.right.out"), W, &L.join_r));
    }
    TM_TRY(to_f32(e, lname(i, "norm1"), W, &L.norm1));
    if (s.mlp) {
        TM_TRY(to_f32(e, lname(i, "norm2"), W, &L.norm2));
        TM_TRY(dense_weight_alloc(L.gu, W, dense_pair_rows(s.ff), dt, st));  // gate and up interleaved: the activation is the GEMM's epilogue
        TM_TRY(place(e, L.gu, 0, 0, lname(i, "mlp.gate"), s.ff, W, 0, 0, false, 1));
        TM_TRY(place(e, L.gu, 0, 0, lname(i, "mlp.up"), s.ff, W, 0, 0, false, 2));
        TM_TRY(dense_weight_alloc(L.down, s.ff, W, dt, st));
        TM_TRY(place(e, L.down, 0, 0, lname(i, "mlp.down"), W, s.ff));
    }
    TM_HIP_CHECK(hipStreamSynchronize(st));
    return 0;
}

static int process_post_layer(tm_engine* e, int i, LmLayer& L, int dt)
{
    const tm_layer_spec& s = L.spec;
    if (s.norm_groups > 0) {
        return process_group_layer(e, i, L, dt);
    }
    const int            W = e->lm->cfg.width, H = s.heads, N = L.c_end;
    TM_TRY(dense_weight_alloc(L.qkv, W, N, dt, e->stream));
    TM_TRY(place(e, L.qkv, 0, 0, lname(i, s.mixer == TM_MIXER_DELTA ? "mix.r" : "mix.q"), L.n_q, W));
    TM_TRY(place(e, L.qkv, L.c_k, 0, lname(i, "mix.k"), L.n_k, W));
    TM_TRY(place(e, L.qkv, L.c_v, 0, lname(i, "mix.v"), L.n_v, W));
    const bool bias = (s.mixer == TM_MIXER_ATTENTION && s.qkv_bias) || s.mixer == TM_MIXER_DELTA;
    if (bias) {
        TM_HIP_CHECK(hipMalloc((void**)&L.proj_bias, (size_t)N * 4));
        TM_HIP_CHECK(hipMemsetAsync(L.proj_bias, 0, (size_t)N * 4, e->stream));
    }
    if (s.mixer == TM_MIXER_ATTENTION) {
        if (s.qkv_bias) {
            TM_TRY(to_f32_at(e, lname(i, "mix.q.b"), L.n_q, L.proj_bias));
            TM_TRY(to_f32_at(e, lname(i, "mix.k.b"), L.n_k, L.proj_bias + L.c_k));
            TM_TRY(to_f32_at(e, lname(i, "mix.v.b"), L.n_v, L.proj_bias + L.c_v));
        }
        if (s.qk_norm_w) {
            TM_TRY(to_f32(e, lname(i, "mix.q.norm"), s.dim, &L.q_w));
            TM_TRY(to_f32(e, lname(i, "mix.k.norm"), s.dim, &L.k_w));
        }
        if (s.rot_dims > 0) {
            std::vector<float> f(s.rot_dims / 2);
            for (int j = 0; j < s.rot_dims / 2; ++j) {
                f[j] = (float)(std::pow((double)s.rot_base, -2.0 * j / s.rot_dims) / (double)s.rot_scale);
            }
            TM_TRY(dmalloc(&L.inv_freq, f.size()));
            TM_HIP_CHECK(hipMemcpyAsync(L.inv_freq, f.data(), f.size() * 4, hipMemcpyHostToDevice, e->stream));
            TM_HIP_CHECK(hipStreamSynchronize(e->stream));
        }
    }
    else {
        TM_TRY(place(e, L.qkv, L.c_g, 0, lname(i, "mix.g"), L.n_att, W));
        TM_TRY(to_f32(e, lname(i, "mix.norm"), L.n_att, &L.mix_norm));
        if (s.mixer == TM_MIXER_LIGHTNING) {
            TM_TRY(dmalloc(&L.decay_d, (size_t)H));
            TM_HIP_CHECK(hipMemcpyAsync(L.decay_d, L.decay_h.data(), (size_t)H * 4, hipMemcpyHostToDevice, e->stream));
            TM_HIP_CHECK(hipStreamSynchronize(e->stream));
        }
        else {
            TM_TRY(place(e, L.qkv, L.c_a, 0, lname(i, "mix.a"), L.n_q, W));
            TM_TRY(place(e, L.qkv, L.c_w1, 0, lname(i, "mix.w1"), s.decay_rank, W));
            TM_TRY(to_f32_at(e, lname(i, "mix.a.b"), L.n_q, L.proj_bias + L.c_a));
            TM_TRY(dense_weight_alloc(L.w2, s.decay_rank, L.n_q, dt, e->stream));
            TM_TRY(place(e, L.w2, 0, 0, lname(i, "mix.w2"), L.n_q, s.decay_rank));
            TM_TRY(to_f32(e, lname(i, "mix.w0"), L.n_q, &L.w0));
        }
    }
    TM_TRY(dense_weight_alloc(L.wo, L.n_att, W, dt, e->stream));
    TM_TRY(place(e, L.wo, 0, 0, lname(i, "mix.o"), W, L.n_att));
    TM_TRY(to_f32(e, lname(i, "norm1"), W, &L.norm1));
    TM_TRY(to_f32(e, lname(i, "norm1.b"), W, &L.norm1_b));
    if (s.mlp) {
        TM_TRY(to_f32(e, lname(i, "norm2"), W, &L.norm2));
        TM_TRY(to_f32(e, lname(i, "norm2.b"), W, &L.norm2_b));
    }
    if (s.mlp == TM_MLP_DENSE) {
        TM_TRY(dense_weight_alloc(L.up, W, s.ff, dt, e->stream));
        TM_TRY(place(e, L.up, 0, 0, lname(i, "mlp.up"), s.ff, W));
        TM_TRY(dense_weight_alloc(L.down, s.ff, W, dt, e->stream));
        TM_TRY(place(e, L.down, 0, 0, lname(i, "mlp.down"), W, s.ff));
        if (s.act == TM_ACT_XIELU) {
            Slot& a = e->slots[lname(i, "mlp.act")];
            TM_REQUIRE(a.filled, "weight not loaded: " + lname(i, "mlp.act"));
            TM_TRY(dmalloc(&L.act_par, (size_t)2));
            xielu_par_kernel<<<1, 64, 0, e->stream>>>(L.act_par, (const uint16_t*)a.dev);
            TM_HIP_CHECK(hipGetLastError());
        }
    }
    else if (s.mlp == TM_MLP_MOE) {
        TM_TRY(dense_weight_alloc(L.router, W, s.experts, dt, e->stream));
        TM_TRY(place(e, L.router, 0, 0, lname(i, "mlp.router"), s.experts, W));
        // a shared expert no larger than the routed ones is one more image of their batched products (zero-padded to their size)
        const int items = s.experts + (L.shared_fused ? 1 : 0);
        TM_TRY(dense_weight_alloc(L.gu, W, s.ff, dt, e->stream, items));
        TM_TRY(dense_weight_alloc(L.down, s.ff, W, dt, e->stream, items));
        for (int x = 0; x < s.experts; ++x) {
            const std::string ex = "mlp.e" + std::to_string(x) + ".";
            TM_TRY(place(e, L.gu, 0, 0, lname(i, (ex + "up").c_str()), s.ff, W, 0, x));
            TM_TRY(place(e, L.down, 0, 0, lname(i, (ex + "down").c_str()), W, s.ff, 0, x));
        }
        if (L.shared_fused) {
            TM_TRY(place(e, L.gu, 0, 0, lname(i, "mlp.shared.up"), s.shared_ff, W, 0, s.experts));
            TM_TRY(place(e, L.down, 0, 0, lname(i, "mlp.shared.down"), W, s.shared_ff, 0, s.experts));
        }
        else if (s.shared_ff > 0) {
            TM_TRY(dense_weight_alloc(L.sh_up, W, s.shared_ff, dt, e->stream));
            TM_TRY(place(e, L.sh_up, 0, 0, lname(i, "mlp.shared.up"), s.shared_ff, W));
            TM_TRY(dense_weight_alloc(L.sh_down, s.shared_ff, W, dt, e->stream));
            TM_TRY(place(e, L.sh_down, 0, 0, lname(i, "mlp.shared.down"), W, s.shared_ff));
        }
    }
    return 0;
}

int layered_process_weights(tm_engine* e)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& c  = lm.cfg;
    const int                dt = c.dtype == TM_DTYPE_F32 ? kDenseF32 : kDenseBf16;
    const int                W  = c.width;
    for (int i = 0; i < c.n_layers; ++i) {
        LmLayer& L = lm.layers[i];
        if (L.src != i) {
            continue;
        }
        const tm_layer_spec& s = L.spec;
        if (L.post) {
            TM_TRY(process_post_layer(e, i, L, dt));
            continue;
        }
        if (L.wide) {
            TM_TRY(process_wide_layer(e, i, L, dt));
            continue;
        }
        TM_TRY(dense_weight_alloc(L.qkv, W, L.n_q + L.n_k + L.n_v, dt, e->stream));
        TM_TRY(place(e, L.qkv, 0, 0, lname(i, "mix.q"), L.n_q, W));
        TM_TRY(place(e, L.qkv, L.n_q, 0, lname(i, "mix.k"), L.n_k, W));
        TM_TRY(place(e, L.qkv, L.n_q + L.n_k, 0, lname(i, "mix.v"), L.n_v, W));
        TM_TRY(dense_weight_alloc(L.out, L.n_att + (s.mlp ? s.ff : 0), W, dt, e->stream));
        // [o | down] along K: the checkpoint rows have their own lengths, each part is placed at its column offset
        TM_TRY(place(e, L.out, 0, 0, lname(i, "mix.o"), W, L.n_att));
        TM_TRY(to_f32(e, lname(i, "norm1"), W, &L.norm1));
        if (s.sink) {
            TM_TRY(to_f32(e, lname(i, "mix.sink"), s.heads, &L.sink));
        }
        if (s.mlp) {
            TM_TRY(dense_weight_alloc(L.up, W, s.ff, dt, e->stream));
            TM_TRY(place(e, L.up, 0, 0, lname(i, "mlp.up"), s.ff, W));
            TM_TRY(place(e, L.out, 0, L.n_att, lname(i, "mlp.down"), W, s.ff));
            TM_TRY(to_f32(e, lname(i, "norm2"), W, &L.norm2));
        }
    }
    for (int i = 0; i < c.n_layers; ++i) {  // borrowed weights
        LmLayer& L = lm.layers[i];
        if (L.src != i) {
            const LmLayer& S = lm.layers[L.src];
            L.qkv = S.qkv, L.up = S.up, L.out = S.out, L.norm1 = S.norm1, L.norm2 = S.norm2, L.sink = S.sink;
            L.wo = S.wo, L.gu = S.gu, L.down = S.down, L.uk = S.uk, L.uv = S.uv;
            L.r1 = S.r1, L.r2 = S.r2, L.rg1_b = S.rg1_b, L.rg2_b = S.rg2_b, L.c_norm = S.c_norm, L.inv_freq = S.inv_freq;
            L.w2 = S.w2, L.router = S.router, L.sh_up = S.sh_up, L.sh_down = S.sh_down, L.norm1_b = S.norm1_b, L.norm2_b = S.norm2_b;
            L.proj_bias = S.proj_bias, L.q_w = S.q_w, L.k_w = S.k_w, L.mix_norm = S.mix_norm, L.w0 = S.w0, L.act_par = S.act_par;
            L.decay_d = S.decay_d;
        }
    }
    if (c.loop_times > 0) {
        TM_TRY(dense_weight_alloc(lm.loop_in, 2 * W, W, dt, e->stream));
        TM_TRY(place(e, lm.loop_in, 0, 0, "loop.in", W, 2 * W));
        TM_TRY(to_f32(e, "loop.step", (size_t)c.loop_times * W, &lm.loop_step));
    }
    TM_TRY(dense_weight_alloc(lm.head, W, c.vocab, dt, e->stream));
    TM_TRY(place(e, lm.head, 0, 0, "head", c.vocab, W));
    TM_TRY(to_f32(e, "final.norm", W, &lm.final_norm));
    if (c.final_layer_norm && c.norm_groups == 0) {
        TM_TRY(to_f32(e, "final.norm.b", W, &lm.final_norm_b));
    }
    {
        Slot& s = e->slots["embed"];
        TM_REQUIRE(s.filled, "weight not loaded: embed");
        if (c.dtype == TM_DTYPE_F32) {
            float* f = nullptr;
            TM_TRY(dmalloc(&f, (size_t)c.vocab * W));
            bf16_to_f32_kernel<<<((size_t)c.vocab * W + 255) / 256, 256, 0, e->stream>>>(f, (const uint16_t*)s.dev, (size_t)c.vocab * W);
            TM_HIP_CHECK(hipGetLastError());
            lm.embed = f;
        }
        else {
            lm.embed = s.dev;  // used in place
            s.dev    = nullptr;
        }
    }
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    for (auto& kv : e->slots) {  // staging is no longer needed
        if (kv.second.dev) {
            (void)hipFree(kv.second.dev);
            kv.second.dev = nullptr;
        }
    }
    e->weights_ready = true;
    return 0;
}

int layered_init_synthetic(tm_engine* e, uint64_t seed)
{
    uint64_t sd = seed * 1000003ull + 29;
    for (auto& kv : e->slots) {
        Slot&             s = kv.second;
        const std::string& n = kv.first;
        if (!s.dev) {
            TM_HIP_CHECK(hipMalloc(&s.dev, s.bytes));
        }
        const size_t cnt  = (size_t)s.bytes / 2;
        const LayeredModel& lm  = *e->lm;
        const size_t        dot = n.rfind('.');
        const std::string   leaf = dot == std::string::npos ? n : n.substr(dot + 1);
        const bool          isnorm = n.find("norm") != std::string::npos;
        const bool          join = leaf == "out" && (n.find("left.out") != std::string::npos || n.find("right.out") != std::string::npos);
        const bool          vec = isnorm || join || leaf == "sink" || leaf == "r1" || leaf == "r2" || (leaf == "b" && n.find("right.b") == std::string::npos)
                                  || leaf == "step" || leaf == "w0" || leaf == "act" || leaf == "lq1" || leaf == "lk1" || leaf == "lq2" || leaf == "lk2"
                                  || leaf == "rel" || leaf == "A_log" || leaf == "dt_bias";
        // matrices: N(0, 1 / in_features) keeps every projection's output at the scale of its input; vectors: small, around zero (norm
        // weights around 1 - norm_offset; distance-penalty numbers positive)
        float stdv = 0.02f, mean = 0.f;
        if ((isnorm && leaf != "b") || join) {
            mean = 1.f - lm.cfg.norm_offset;
        }
        else if (leaf == "r1" || leaf == "r2") {
            mean = 0.5f;
        }
        if (!vec && n != "embed") {
            int  K  = lm.cfg.width;
            auto fi = lm.fan_in.find(n);
            if (fi != lm.fan_in.end()) {
                K = fi->second;
            }
            else if (leaf == "o" || leaf == "down") {
                K = (int)(cnt / lm.cfg.width);
            }
            stdv = 1.0f / std::sqrt((float)K);
        }
        else if (n == "embed") {
            stdv = 1.0f;
        }
        fill_normal_bf16_kernel<<<(cnt + 255) / 256, 256, 0, e->stream>>>((uint16_t*)s.dev, cnt, mean, stdv, ++sd);
        TM_HIP_CHECK(hipGetLastError());
        s.filled = true;
    }
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    return 0;
}

template<class T>
static int lm_alloc(T** p, size_t n, hipStream_t st)
{
    TM_HIP_CHECK(hipMalloc((void**)p, n * sizeof(T)));
    TM_HIP_CHECK(hipMemsetAsync(*p, 0, n * sizeof(T), st));
    return 0;
}

// start-up allocation of a layer-list engine: activation buffers, batch state, block pool (the engine's own fields, so that the
// static batch, continuous batching and the sampler run unchanged)
int layered_start(tm_engine* e)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    const tm_engine_config&  c  = e->cfg;
    hipStream_t              st = e->stream;
    const int                B  = c.max_batch_size;
    e->max_blocks_per_seq = (c.session_len + c.cache_block_seq_len - 1) / c.cache_block_seq_len;
    e->max_tokens         = std::max(B, std::max(64, c.max_prefill_token_num));
    const size_t T        = e->max_tokens;
    // cache block: every layer run has its keys [kv_heads][block_len][dim] and, behind them, its values transposed [kv_heads][vdim][block_len]
    lm.ldw      = (m.width + 31) / 32 * 32;
    int64_t off = 0;
    int     max_qkv = 8, max_cat = 32, max_vdim = 0, max_heads = 0;
    int     max_proj = 0, max_q = 0, max_plain = 0, max_lat = 0, max_ff = 0;
    bool    any_moe = false;
    int     max_mix = 0, max_lora = 0, max_conv = 0;
    bool    any_join = false;
    for (LmLayer& L : lm.layers) {
        const bool stateful = L.has_state;
        const bool parallel = L.spec.mixer == TM_MIXER_PARALLEL;
        if (stateful) {  // a recurrent state per slot (instead of cache entries, or beside them)
            L.state_offset = lm.state_slot_floats;
            L.state_floats = parallel ? state_mix_floats(L.spec.r_heads, L.spec.r_dim, L.spec.r_vdim) : state_mix_floats(L.spec.heads, L.spec.dim, L.spec.vdim);
            lm.state_slot_floats += L.state_floats;
            max_mix  = std::max(max_mix, parallel ? std::max(L.r_nv, L.spec.r_heads * L.spec.r_dim) : L.n_att);
            max_lora = std::max(max_lora, parallel ? L.lora_g1 + L.g2.Kp : L.w2.Kp);
        }
        if (L.conv_taps > 0) {  // the last taps - 1 inputs of a short convolution are state too
            L.conv_offset = lm.state_slot_floats;
            L.conv_floats = (size_t)(L.conv_taps - 1) * L.conv_ch;
            lm.state_slot_floats += L.conv_floats;
            max_conv = std::max(max_conv, L.conv_ch + (parallel ? 2 * L.spec.r_heads * L.spec.r_dim : 0));
        }
        if (L.has_cache) {
            L.kv_offset = off;
            L.v_offset  = (int64_t)L.n_k * c.cache_block_seq_len * lm.elem;
            off += (int64_t)(L.n_k + L.n_v) * c.cache_block_seq_len * lm.elem;
            off         = (off + 15) / 16 * 16;
            max_vdim    = std::max(max_vdim, L.a_vdim);
            max_heads   = std::max(max_heads, L.a_heads);
        }
        if (L.post && L.spec.norm_groups > 0) {  // the attention output stays fp32 until the heads are joined / gated
            max_mix  = std::max(max_mix, L.a_heads * L.a_vdim);
            max_cat  = std::max(max_cat, L.wo_r.Kp);
            any_join = any_join || parallel;
        }
        if (L.post) {
            max_cat  = std::max(max_cat, L.wo.Kp);
            max_proj = std::max(max_proj, std::max(L.qkv.N, L.spec.experts));
            max_q    = std::max(max_q, L.has_cache ? L.a_heads * L.a_dim : 0);
            if (L.spec.mlp) {
                max_ff     = std::max(max_ff, std::max(L.down.Kp, L.sh_down.Kp));
                lm.max_top = std::max(lm.max_top, L.spec.mlp == TM_MLP_MOE ? L.spec.top + (L.shared_fused ? 1 : 0) : 1);
                any_moe    = any_moe || L.spec.mlp == TM_MLP_MOE;
            }
            continue;
        }
        if (!L.wide) {
            max_qkv = std::max(max_qkv, L.qkv.N);
            max_cat = std::max(max_cat, L.out.Kp);
            continue;
        }
        max_cat   = std::max(max_cat, L.wo.Kp);
        max_proj  = std::max(max_proj, L.qkv.N);
        max_q     = std::max(max_q, L.spec.heads * L.a_dim);
        max_plain = std::max(max_plain, L.spec.heads * L.plain_stride);
        max_lat   = std::max(max_lat, L.spec.heads * L.lat_stride);
        if (L.spec.mlp) {
            max_ff     = std::max(max_ff, L.down.Kp);
            lm.max_top = std::max(lm.max_top, L.spec.mlp == TM_MLP_MOE ? L.spec.top : 1);
            any_moe    = any_moe || L.spec.mlp == TM_MLP_MOE;
        }
    }
    e->block_bytes = std::max<int64_t>(off, 16);  // (a model without attention layers still has a block pool: the scheduler counts tokens in blocks)
    max_vdim = std::max(max_vdim, 1), max_heads = std::max(max_heads, 1);
    lm.ldqkv = (max_qkv + 31) / 32 * 32;
    lm.ldcat = max_cat;
    lm.ldv16 = e->vocab_local;
    lm.max_logit_rows = (int)std::max<size_t>(B, std::min<size_t>(T, 1024));
    if (max_proj > 0) {  // wide blocks
        const size_t TT = T * std::max(1, lm.max_top);  // rows of the experts' products: one per (token, chosen expert)
        lm.ldproj  = (max_proj + 3) / 4 * 4;
        lm.ldq     = std::max(32, (max_q + 31) / 32 * 32);
        lm.ldplain = std::max(32, max_plain);
        lm.ldlat   = std::max(32, max_lat);
        lm.ldff    = std::max(32, max_ff);
        TM_TRY(lm_alloc(&lm.d_proj, T * lm.ldproj, st));
        TM_TRY(lm_alloc((char**)&lm.d_q, T * lm.ldq * lm.elem, st));
        TM_TRY(lm_alloc((char**)&lm.d_plain, T * lm.ldplain * lm.elem, st));
        TM_TRY(lm_alloc((char**)&lm.d_lat, T * lm.ldlat * lm.elem, st));
        TM_TRY(lm_alloc((char**)&lm.d_ff, TT * lm.ldff * lm.elem, st));
        if (any_moe) {
            TM_TRY(lm_alloc((char**)&lm.d_moe_x, TT * lm.ldw * lm.elem, st));
            TM_TRY(lm_alloc(&lm.d_moe_y, TT * m.width, st));
            TM_TRY(lm_alloc(&lm.d_topk_w, TT, st));
            TM_TRY(lm_alloc(&lm.d_topk_ids, TT, st));
            TM_TRY(lm_alloc(&lm.d_f2n, TT, st));
            TM_TRY(lm_alloc(&lm.d_en2f, TT, st));
            TM_TRY(lm_alloc(&lm.d_offsets, (size_t)1026, st));
        }
    }
    if (m.loop_times > 0) {
        lm.ld2w = lm.loop_in.Kp;
        TM_TRY(lm_alloc(&lm.d_x0, T * m.width, st));
        TM_TRY(lm_alloc((char**)&lm.d_xx, T * lm.ld2w * lm.elem, st));
    }
    if (lm.has_post) {
        lm.ldmix  = std::max(4, (max_mix + 3) / 4 * 4);
        lm.ldlora = std::max(32, max_lora);
        TM_TRY(lm_alloc(&lm.d_y, T * m.width, st));
        TM_TRY(lm_alloc(&lm.d_mixo, T * lm.ldmix, st));
        TM_TRY(lm_alloc(&lm.d_aux, T * lm.ldmix, st));
        TM_TRY(lm_alloc(&lm.d_wdec, T * lm.ldmix, st));
        TM_TRY(lm_alloc((char**)&lm.d_lora, T * lm.ldlora * lm.elem, st));
        if (max_conv > 0) {
            lm.ldconv = (max_conv + 3) / 4 * 4;
            TM_TRY(lm_alloc(&lm.d_conv, T * lm.ldconv, st));
        }
        if (any_join) {
            TM_TRY(lm_alloc(&lm.d_y2, T * m.width, st));
            TM_TRY(lm_alloc(&lm.d_gate2, T * lm.ldmix, st));
        }
    }
    if (lm.state_slot_floats > 0) {
        TM_TRY(lm_alloc(&lm.d_state, ((size_t)B + 1) * lm.state_slot_floats, st));
    }
    TM_TRY(lm_alloc(&lm.d_res, T * m.width, st));
    TM_TRY(lm_alloc((char**)&lm.d_h1, T * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_h2, T * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_qkv, T * lm.ldqkv * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_cat, T * lm.ldcat * lm.elem, st));
    TM_TRY(lm_alloc((char**)&lm.d_hn, (size_t)lm.max_logit_rows * lm.ldw * lm.elem, st));
    TM_TRY(lm_alloc(&lm.d_logits_f32, (size_t)lm.max_logit_rows * m.vocab, st));
    TM_TRY(lm_alloc(&lm.d_row_seq, T, st));
    TM_TRY(lm_alloc(&lm.d_row_pos, T, st));
    TM_TRY(lm_alloc(&lm.d_want, T, st));
    TM_TRY(lm_alloc(&lm.d_iota, T, st));
    TM_TRY(lm_alloc(&lm.d_seq_slot, (size_t)B, st));
    TM_TRY(lm_alloc(&lm.d_step_ids, T, st));
    TM_TRY(lm_alloc(&lm.d_step_cu_q, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&lm.d_step_k_len, (size_t)B, st));
    iota_kernel<<<(T + 255) / 256, 256, 0, st>>>(lm.d_iota, (int)T);
    TM_HIP_CHECK(hipGetLastError());
    // decode rows split their keys so that a few long sequences still fill the device: >= 4 cache blocks per split at full length
    lm.decode_splits = std::min(8, std::max(1, e->max_blocks_per_seq / 4));
    lm.attn_ws_bytes = general_attention_workspace_bytes(B, max_heads, max_vdim, lm.decode_splits);
    TM_HIP_CHECK(hipMalloc((void**)&lm.d_attn_ws, lm.attn_ws_bytes));

    // the engine's batch state (same fields as every other model family)
    TM_TRY(lm_alloc(&e->d_logits, (size_t)B * e->vocab_local, st));
    TM_TRY(lm_alloc(&e->d_ids, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_next_ids, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_k_len, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_cu_q, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_cu_q_b, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_cu_koff, (size_t)B + 1, st));
    TM_TRY(lm_alloc(&e->d_rows, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_generated, (size_t)B * c.session_len, st));
    TM_TRY(lm_alloc(&e->d_step, (size_t)1, st));
    TM_TRY(lm_alloc(&e->d_prefill_ids, T, st));
    TM_TRY(lm_alloc(&e->d_argmax_val, (size_t)B, st));
    TM_TRY(lm_alloc(&e->d_cand, (size_t)B * 2, st));
    TM_TRY(lm_alloc(&e->d_cand_all, (size_t)B * 2, st));
    TM_TRY(lm_alloc(&e->d_block_ptrs, (size_t)B * e->max_blocks_per_seq, st));
    TM_TRY(lm_alloc(&e->d_cu_block_nums, (size_t)B + 1, st));
    e->kflat_stride = 1 << 30;  // no flatten scratch in this family: the attention kernels read the paged cache

    int64_t blocks = c.cache_blocks;
    if (blocks <= 0) {
        size_t free_b = 0, total_b = 0;
        TM_HIP_CHECK(hipMemGetInfo(&free_b, &total_b));
        const float frac = c.cache_max_entry_count > 0.f ? c.cache_max_entry_count : 0.8f;
        blocks           = (int64_t)((double)free_b * frac / (double)e->block_bytes);
        blocks           = std::min(blocks, (int64_t)B * e->max_blocks_per_seq + 1);
    }
    TM_REQUIRE(blocks >= 1, "no memory for KV blocks");
    if (hipMalloc((void**)&e->pool, (size_t)blocks * e->block_bytes) != hipSuccess) {
        (void)hipGetLastError();
        set_last_error("KV pool allocation failed");
        return TM_OOM;
    }
    TM_HIP_CHECK(hipMemsetAsync(e->pool, 0, (size_t)blocks * e->block_bytes, st));
    e->num_blocks = blocks;
    e->free_blocks.resize(blocks);
    for (int64_t i = 0; i < blocks; ++i) {
        e->free_blocks[i] = (int)(blocks - 1 - i);
    }
    TM_HIP_CHECK(hipStreamSynchronize(st));
    e->started = true;
    return 0;
}

void layered_free(tm_engine* e)
{
    if (!e->lm) {
        return;
    }
    LayeredModel& lm = *e->lm;
    for (size_t i = 0; i < lm.layers.size(); ++i) {
        LmLayer& L = lm.layers[i];
        if (L.src == (int)i) {
            dense_weight_free(L.qkv), dense_weight_free(L.up), dense_weight_free(L.out);
            dense_weight_free(L.wo), dense_weight_free(L.gu), dense_weight_free(L.down), dense_weight_free(L.uk), dense_weight_free(L.uv);
            dense_weight_free(L.w2), dense_weight_free(L.router), dense_weight_free(L.sh_up), dense_weight_free(L.sh_down);
            dense_weight_free(L.wo_r), dense_weight_free(L.a2), dense_weight_free(L.g2);
            for (float* p : {L.norm1, L.norm2, L.sink, L.r1, L.r2, L.rg1_b, L.rg2_b, L.c_norm, L.inv_freq, L.norm1_b, L.norm2_b, L.proj_bias,
                             L.q_w, L.k_w, L.mix_norm, L.w0, L.act_par, L.decay_d, L.conv_w, L.lambda, L.dist_tab, L.talk, L.zero_sink, L.join_l,
                             L.join_r, L.a_log, L.dt_bias, L.r_norm}) {
                if (p) {
                    (void)hipFree(p);
                }
            }
        }
    }
    dense_weight_free(lm.head);
    dense_weight_free(lm.loop_in);
    for (void* p : {(void*)lm.d_y, (void*)lm.d_mixo, (void*)lm.d_aux, (void*)lm.d_wdec, lm.d_lora, (void*)lm.d_state, (void*)lm.final_norm_b,
                    (void*)lm.d_y2, (void*)lm.d_conv, (void*)lm.d_gate2}) {
        if (p) {
            (void)hipFree(p);
        }
    }
    for (void* p : {(void*)lm.loop_step, (void*)lm.d_proj, (void*)lm.d_x0, (void*)lm.d_moe_y, (void*)lm.d_topk_w, lm.d_q, lm.d_plain, lm.d_lat,
                    lm.d_ff, lm.d_xx, lm.d_moe_x, (void*)lm.d_topk_ids, (void*)lm.d_offsets, (void*)lm.d_f2n, (void*)lm.d_en2f}) {
        if (p) {
            (void)hipFree(p);
        }
    }
    for (void* p : {(void*)lm.embed, (void*)lm.final_norm, (void*)lm.d_res, lm.d_h1, lm.d_h2, lm.d_qkv, lm.d_cat, lm.d_hn, (void*)lm.d_logits_f32,
                    (void*)lm.d_row_seq, (void*)lm.d_row_pos, (void*)lm.d_iota, (void*)lm.d_want, (void*)lm.d_seq_slot, (void*)lm.d_step_ids,
                    (void*)lm.d_step_cu_q, (void*)lm.d_step_k_len, (void*)lm.d_attn_ws}) {
        if (p) {
            (void)hipFree(p);
        }
    }
}

// ---- forward ------------------------------------------------------------------------------------------------------------------------
static GeneralAttnParams attn_params(tm_engine* e, const LmLayer& L, const LmPart& P)
{
    LayeredModel&     lm = *e->lm;
    GeneralAttnParams p{};
    p.q            = (const char*)lm.d_qkv + (size_t)P.row0 * lm.ldqkv * lm.elem;
    p.out          = (char*)lm.d_cat + (size_t)P.row0 * lm.ldcat * lm.elem;
    p.ldq          = lm.ldqkv;
    p.ldo          = lm.ldcat;
    if (L.wide || L.post) {
        p.q   = (const char*)lm.d_q + (size_t)P.row0 * lm.ldq * lm.elem;
        p.ldq = lm.ldq;
        if (L.spec.mixer == TM_MIXER_LATENT) {  // the attention output stays in the latent space until the value expansion
            p.out             = (char*)lm.d_lat + (size_t)P.row0 * lm.ldlat * lm.elem;
            p.ldo             = lm.ldlat;
            p.out_head_stride = L.lat_stride;
        }
        if (L.spec.out_gate) {
            p.out_gate = lm.d_proj + (size_t)P.row0 * lm.ldproj + L.c_g;
            p.ld_gate  = lm.ldproj;
        }
        if (L.post && L.spec.norm_groups > 0 && (L.spec.diff_maps || L.spec.mixer == TM_MIXER_PARALLEL)) {
            p.out     = lm.d_mixo + (size_t)P.row0 * lm.ldmix;  // fp32 until the maps are joined / the gate is applied
            p.ldo     = lm.ldmix;
            p.out_f32 = 1;
        }
    }
    p.k_heads        = L.a_kh;
    p.v_heads        = L.a_vh;
    p.dist_table     = L.dist_tab;
    p.dist_table_len = L.dist_len;
    p.dist_r1 = L.r1;
    p.dist_r2 = L.r2;
    p.chunk   = L.spec.chunk;
    p.window  = L.spec.window;
    p.keep_first = L.spec.keep_first;
    p.rows         = P.rows;
    p.row_seq      = lm.d_row_seq + P.row0;
    p.row_pos      = lm.d_row_pos + P.row0;
    p.seq_slot     = P.seq_slot;
    p.block_ptrs   = P.block_ptrs;
    p.block_stride = e->max_blocks_per_seq;
    p.layer_offset = L.kv_offset;
    p.v_offset     = L.v_offset;
    p.block_len    = e->cfg.cache_block_seq_len;
    p.elem_bytes   = lm.elem;
    p.q_heads      = L.a_heads;
    p.kv_heads     = L.a_kv;
    p.dim          = L.a_dim;
    p.vdim         = L.a_vdim;
    p.scale        = L.spec.scale;
    p.softcap      = L.spec.softcap;
    p.qtemp_coef   = L.spec.qtemp_coef;
    p.qtemp_every  = L.spec.qtemp_every;
    p.sink         = L.sink ? L.sink : L.zero_sink;
    p.nseq         = P.nseq;
    p.max_q_len    = P.max_q_len;
    p.cu_q         = P.cu_q;
    p.k_len        = P.k_len;
    return p;
}

// one wide block over M rows (see the head of this file)
static int wide_layer(tm_engine* e, const LmLayer& L, int M, const LmPart* parts, int nparts)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    const tm_layer_spec&     s  = L.spec;
    hipStream_t              st = e->stream;
    const int                W = m.width, H = s.heads;
    const bool               latent = s.mixer == TM_MIXER_LATENT;
    TM_PROF(P_RES_NORM, TM_TRY(launch_rmsnorm_f32(lm.d_h1, nullptr, lm.ldw, lm.elem, lm.d_res, nullptr, L.norm1, nullptr, m.norm_offset, m.norm_eps,
                                                  M, W, st)));
    TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_linear(L.qkv, lm.d_h1, lm.ldw, lm.d_proj, lm.ldproj, M, kDenseScaleF32, 1.f, st)));
    for (int i = 0; i < nparts; ++i) {
        const LmPart&     P    = parts[i];
        GeneralAttnParams p    = attn_params(e, L, P);
        const float*      proj = lm.d_proj + (size_t)P.row0 * lm.ldproj;
        if (latent) {
            TM_PROF(P_KV_STORE, TM_TRY(launch_latent_prep(proj, lm.ldproj, 0, L.c_k, (char*)lm.d_plain + (size_t)P.row0 * lm.ldplain * lm.elem, lm.ldplain,
                                                          L.plain_stride, (void*)p.q, lm.ldq, L.c_norm, L.inv_freq, s.dim, s.rot_dim, s.kv_rank,
                                                          s.rot_dims > 0 ? s.rot_dims : s.rot_dim, m.norm_eps, p, st)));
        }
        else {
            TM_PROF(P_KV_STORE, TM_TRY(launch_attn_prep(proj, lm.ldproj, 0, L.c_k, L.c_v, (void*)p.q, lm.ldq, s.qk_unit_norm != 0, s.v_unit_norm != 0,
                                                        m.norm_eps, p, st)));
        }
    }
    if (latent) {
        DenseCall c;
        c.count        = H;
        c.x_col_stride = L.plain_stride;
        c.y_col_stride = L.a_dim;
        TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_call(L.uk, lm.d_plain, lm.ldplain, lm.d_q, lm.ldq, M, c, st)));
    }
    for (int i = 0; i < nparts; ++i) {
        const LmPart&     P = parts[i];
        GeneralAttnParams p = attn_params(e, L, P);
        if (P.decode && lm.decode_splits > 1 && general_attention_workspace_bytes(P.rows, H, L.a_vdim, lm.decode_splits) <= lm.attn_ws_bytes) {
            p.splits     = lm.decode_splits;
            p.partial_o  = lm.d_attn_ws;
            p.partial_ml = lm.d_attn_ws + (size_t)P.rows * H * p.splits * L.a_vdim;
        }
        TM_PROF(P_ATTN, TM_TRY(launch_general_attention(p, !P.decode, st)));
    }
    if (latent) {
        DenseCall c;
        c.count        = H;
        c.x_col_stride = L.lat_stride;
        c.y_col_stride = s.vdim;
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_call(L.uv, lm.d_lat, lm.ldlat, lm.d_cat, lm.ldcat, M, c, st)));
    }
    DenseCall close;  // the sublayer's result joins the stream: gated element by element, or scaled
    close.epi   = s.resid_gate ? kDenseResidGate : kDenseResidAdd;
    close.alpha = m.residual_mult;
    close.ldg   = lm.ldproj;
    if (s.resid_gate) {
        close.gate      = lm.d_proj + L.c_rg1;
        close.gate_bias = L.rg1_b;
    }
    TM_PROF(P_GEMM_O, TM_TRY(launch_dense_call(L.wo, lm.d_cat, lm.ldcat, lm.d_res, W, M, close, st)));
    if (s.resid_gate) {
        close.gate      = lm.d_proj + L.c_rg2;
        close.gate_bias = L.rg2_b;
    }
    if (s.mlp == TM_MLP_GATED) {
        DenseCall c;  // act(gate) * up leaves the [gate | up] product's epilogue in the activation type
        c.epi   = kDenseGatedAct;
        c.act   = s.act;
        c.n_out = s.ff;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_call(L.gu, lm.d_h1, lm.ldw, lm.d_ff, lm.ldff, M, c, st)));
        TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_call(L.down, lm.d_ff, lm.ldff, lm.d_res, W, M, close, st)));
    }
    else if (s.mlp == TM_MLP_MOE) {
        const int k = s.top, E = s.experts;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_topk_sigmoid(lm.d_topk_ids, lm.d_topk_w, lm.d_proj + L.c_router, lm.ldproj, M, E, k, st)));
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_route(lm.d_offsets, lm.d_f2n, lm.d_en2f, lm.d_topk_ids, M, E, k, st)));
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_gather(lm.d_moe_x, lm.ldw, lm.d_h1, lm.ldw, lm.elem, lm.d_topk_w, lm.d_en2f, M, W, k, true, st)));
        DenseCall c;
        c.epi         = kDenseGatedAct;
        c.act         = s.act;
        c.n_out       = s.ff;
        c.count       = E;
        c.row_offsets = lm.d_offsets;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_call(L.gu, lm.d_moe_x, lm.ldw, lm.d_ff, lm.ldff, M * k, c, st)));
        c.epi = kDenseScaleF32;
        TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_call(L.down, lm.d_ff, lm.ldff, lm.d_moe_y, W, M * k, c, st)));
        TM_PROF(P_GEMM_DOWN, TM_TRY(launch_moe_combine_f32(lm.d_res, lm.d_moe_y, lm.d_topk_w, lm.d_en2f, s.resid_gate ? close.gate : nullptr, lm.ldproj,
                                                     close.gate_bias, M, W, k, false, st)));
    }
    return 0;
}

// the sequences of a part as the state kernels read them; the caller sets layer_offset
static StateMixParams state_seqs(tm_engine* e, const LmPart& P)
{
    LayeredModel&  lm = *e->lm;
    StateMixParams sp;
    sp.max_q_len = P.decode ? 1 : std::max(1, P.max_q_len);
    sp.nseq = P.nseq, sp.cu_q = P.cu_q, sp.k_len = P.k_len, sp.seq_slot = P.seq_slot, sp.slot0 = P.slot0, sp.active = P.active;
    sp.park_slot   = e->cfg.max_batch_size;
    sp.state       = lm.d_state;
    sp.slot_stride = lm.state_slot_floats;
    return sp;
}

static int run_attention_parts(tm_engine* e, const LmLayer& L, const LmPart* parts, int nparts)
{
    LayeredModel& lm = *e->lm;
    for (int i = 0; i < nparts; ++i) {
        const LmPart&     P = parts[i];
        GeneralAttnParams p = attn_params(e, L, P);
        if (P.decode && lm.decode_splits > 1 && general_attention_workspace_bytes(P.rows, L.a_heads, L.a_vdim, lm.decode_splits) <= lm.attn_ws_bytes) {
            p.splits     = lm.decode_splits;
            p.partial_o  = lm.d_attn_ws;
            p.partial_ml = lm.d_attn_ws + (size_t)P.rows * L.a_heads * p.splits * L.a_vdim;
        }
        TM_PROF(P_ATTN, TM_TRY(launch_general_attention(p, !P.decode, e->stream)));
    }
    return 0;
}

// one post-norm block with RMS group norms over M rows (see the head of this file); lm.d_h1 holds the stream in the activation type
static int group_layer(tm_engine* e, const LmLayer& L, int M, const LmPart* parts, int nparts)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    const tm_layer_spec&     s  = L.spec;
    hipStream_t              st = e->stream;
    const int                W = m.width, H = s.heads, groups = s.norm_groups;
    TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_linear(L.qkv, lm.d_h1, lm.ldw, lm.d_proj, lm.ldproj, M, kDenseScaleF32, 1.f, st)));
    if (L.conv_taps > 0) {
        for (int i = 0; i < nparts; ++i) {
            const LmPart&  P  = parts[i];
            if (P.decode && s.mixer == TM_MIXER_ATTENTION) {
                continue;  // decoded tokens: the convolution runs inside the prepare kernel (one row per sequence)
            }
            StateMixParams sp = state_seqs(e, P);
            sp.layer_offset   = L.conv_offset;
            TM_PROF(P_KV_STORE, TM_TRY(launch_short_conv(lm.d_conv + (size_t)P.row0 * lm.ldconv, lm.ldconv, lm.d_proj + (size_t)P.row0 * lm.ldproj, lm.ldproj,
                                                         L.conv_col, L.conv_w, L.conv_ch, L.conv_taps, L.conv_act, sp, st)));
        }
    }
    if (s.mixer == TM_MIXER_ATTENTION) {
        const float* src = L.conv_taps > 0 ? lm.d_conv : lm.d_proj;  // (the convolved columns start at column 0 of both)
        const int    ld  = L.conv_taps > 0 ? lm.ldconv : lm.ldproj;
        AttnPrepExtra ex;
        ex.q_w = L.q_w, ex.k_w = L.k_w, ex.inv_freq = L.inv_freq, ex.rot_dims = s.rot_dims;
        ex.maps = s.diff_maps ? 2 : 1, ex.rot_pairs = s.rot_pairs;
        ex.rot_mult = s.yarn_factor > 0.f ? 0.1f * std::log(s.yarn_factor) + 1.f : 1.f;
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            AttnPrepExtra     px = ex;
            const bool        fused = P.decode && L.conv_taps > 0;
            if (fused) {
                px.conv_w = L.conv_w, px.conv_taps = L.conv_taps, px.conv_ch = L.conv_ch;
                px.conv_state = lm.d_state, px.conv_slot_stride = lm.state_slot_floats, px.conv_offset = L.conv_offset;
                px.conv_slot0 = P.slot0, px.conv_park_slot = e->cfg.max_batch_size, px.conv_active = P.active;
            }
            const float* from = fused ? lm.d_proj : src;
            const int    ldf  = fused ? lm.ldproj : ld;
            TM_PROF(P_KV_STORE, TM_TRY(launch_attn_prep(from + (size_t)P.row0 * ldf, ldf, 0, L.c_k, L.c_v, (void*)p.q, lm.ldq, s.qk_norm_w != 0, false,
                                                        m.norm_eps, p, st, px)));
        }
        TM_TRY(run_attention_parts(e, L, parts, nparts));
        if (s.diff_maps) {
            TM_PROF(P_ATTN, TM_TRY(launch_diff_head_norm(lm.d_cat, lm.ldcat, lm.elem, lm.d_mixo, lm.ldmix, L.lambda, 1.f - s.diff_init, M, H, s.vdim,
                                                         m.norm_eps, st)));
        }
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.wo, lm.d_cat, lm.ldcat, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
        TM_PROF(P_RES_NORM, TM_TRY(launch_group_rmsnorm_add_f32(lm.d_res, lm.d_h1, lm.ldw, lm.elem, lm.d_y, nullptr, nullptr, nullptr, L.norm1, groups,
                                                                m.norm_eps, M, W, st)));
    }
    else {
        // ---- left: attention with mixed heads, distance table, zero sink, output gate ----
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            TM_PROF(P_KV_STORE, TM_TRY(launch_talk_prep(lm.d_proj + (size_t)P.row0 * lm.ldproj, lm.ldproj, 0, L.c_k, (void*)p.q, lm.ldq, L.q_w, L.k_w, L.talk,
                                                        s.dim, m.norm_eps, p, st)));
        }
        TM_TRY(run_attention_parts(e, L, parts, nparts));
        TM_PROF(P_ATTN, TM_TRY(launch_sigmoid_gate_mul(lm.d_cat, lm.ldcat, lm.elem, lm.d_mixo, lm.ldmix, lm.d_proj + L.c_g, lm.ldproj, M, L.n_att, st)));
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.wo, lm.d_cat, lm.ldcat, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
        // ---- right: gated delta rule ----
        const int Hr = s.r_heads, dr = s.r_dim, dvr = s.r_vdim;
        TM_PROF(P_KV_STORE, TM_TRY(launch_act_cast_f32(lm.d_lora, lm.ldlora, lm.elem, lm.d_proj + L.c_a1, lm.ldproj, M, L.lora_g1 + s.g_rank, 0, st)));
        DenseCall c;
        c.epi  = kDenseBiasF32;
        c.bias = L.dt_bias;
        TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_call(L.a2, lm.d_lora, lm.ldlora, lm.d_wdec, lm.ldmix, M, c, st)));
        TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_linear(L.g2, (const char*)lm.d_lora + (size_t)L.lora_g1 * lm.elem, lm.ldlora, lm.d_gate2, lm.ldmix, M,
                                                       kDenseScaleF32, 1.f, st)));
        TM_PROF(P_KV_STORE, TM_TRY(launch_gdelta_prep(lm.d_conv, lm.ldconv, 0, L.r_nqk, L.c_xq, L.c_xk, lm.d_proj + L.c_b, lm.ldproj, lm.d_wdec, lm.ldmix,
                                                      L.a_log, nullptr, lm.d_aux, lm.ldmix, M, Hr, s.r_kv_heads, dr, st)));
        for (int i = 0; i < nparts; ++i) {
            const LmPart&  P  = parts[i];
            StateMixParams sp = state_seqs(e, P);
            sp.layer_offset   = L.state_offset;
            sp.heads = Hr, sp.dim = dr, sp.vdim = dvr;
            sp.proj = lm.d_conv + (size_t)P.row0 * lm.ldconv, sp.ld = lm.ldconv;
            sp.c_q = L.c_xq, sp.c_k = L.c_xk, sp.c_a = L.c_xk, sp.c_v = 2 * L.r_nqk;
            sp.decay_w = lm.d_wdec + (size_t)P.row0 * lm.ldmix, sp.ld_w = lm.ldmix;
            sp.unit    = lm.d_aux + (size_t)P.row0 * lm.ldmix, sp.ld_u = lm.ldmix;
            sp.out     = lm.d_mixo + (size_t)P.row0 * lm.ldmix, sp.ldo = lm.ldmix;
            TM_PROF(P_ATTN, TM_TRY(launch_state_mix(sp, true, st)));
        }
        TM_PROF(P_ATTN, TM_TRY(launch_gated_group_norm(lm.d_cat, lm.ldcat, lm.elem, lm.d_mixo, lm.ldmix, L.r_norm, lm.d_gate2, lm.ldmix, M, Hr, dvr,
                                                       m.norm_eps, st)));
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.wo_r, lm.d_cat, lm.ldcat, lm.d_y2, W, M, kDenseScaleF32, 1.f, st)));
        TM_PROF(P_RES_NORM, TM_TRY(launch_group_rmsnorm_add_f32(lm.d_res, lm.d_h1, lm.ldw, lm.elem, lm.d_y, lm.d_y2, L.join_l, L.join_r, L.norm1, groups,
                                                                m.norm_eps, M, W, st)));
    }
    if (s.mlp == TM_MLP_NONE) {
        return 0;
    }
    DenseCall c;  // act(gate) * up leaves the [gate | up] product's epilogue in the activation type
    c.epi   = kDenseGatedAct;
    c.act   = s.act;
    c.n_out = s.ff;
    TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_call(L.gu, lm.d_h1, lm.ldw, lm.d_ff, lm.ldff, M, c, st)));
    TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_linear(L.down, lm.d_ff, lm.ldff, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
    TM_PROF(P_RES_NORM, TM_TRY(launch_group_rmsnorm_add_f32(lm.d_res, lm.d_h1, lm.ldw, lm.elem, lm.d_y, nullptr, nullptr, nullptr, L.norm2, groups,
                                                            m.norm_eps, M, W, st)));
    return 0;
}

// one post-norm block over M rows (see the head of this file); h_ready: lm.d_h1 already holds the stream in the activation type
static int post_layer(tm_engine* e, const LmLayer& L, int M, const LmPart* parts, int nparts, bool h_ready)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    const tm_layer_spec&     s  = L.spec;
    hipStream_t              st = e->stream;
    const int                W = m.width, H = s.heads;
    if (!h_ready) {
        TM_PROF(P_RES_NORM, TM_TRY(launch_act_cast_f32(lm.d_h1, lm.ldw, lm.elem, lm.d_res, W, M, W, 0, st)));
    }
    if (s.norm_groups > 0) {
        return group_layer(e, L, M, parts, nparts);
    }
    DenseCall pc;
    pc.epi  = L.proj_bias ? kDenseBiasF32 : kDenseScaleF32;
    pc.bias = L.proj_bias;
    TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_call(L.qkv, lm.d_h1, lm.ldw, lm.d_proj, lm.ldproj, M, pc, st)));
    if (s.mixer == TM_MIXER_ATTENTION) {
        AttnPrepExtra ex;
        ex.q_w = L.q_w, ex.k_w = L.k_w, ex.inv_freq = L.inv_freq, ex.rot_dims = s.rot_dims;
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            TM_PROF(P_KV_STORE, TM_TRY(launch_attn_prep(lm.d_proj + (size_t)P.row0 * lm.ldproj, lm.ldproj, 0, L.c_k, L.c_v, (void*)p.q, lm.ldq,
                                                        s.qk_norm_w != 0, false, m.norm_eps, p, st, ex)));
        }
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            if (P.decode && lm.decode_splits > 1 && general_attention_workspace_bytes(P.rows, H, L.a_vdim, lm.decode_splits) <= lm.attn_ws_bytes) {
                p.splits     = lm.decode_splits;
                p.partial_o  = lm.d_attn_ws;
                p.partial_ml = lm.d_attn_ws + (size_t)P.rows * H * p.splits * L.a_vdim;
            }
            TM_PROF(P_ATTN, TM_TRY(launch_general_attention(p, !P.decode, st)));
        }
    }
    else {
        const bool delta = s.mixer == TM_MIXER_DELTA;
        if (delta) {  // decay logits = w2 tanh(w1 h) + w0; then unit keys, removal rates and decays as the recurrence reads them
            TM_PROF(P_KV_STORE, TM_TRY(launch_act_cast_f32(lm.d_lora, lm.ldlora, lm.elem, lm.d_proj + L.c_w1, lm.ldproj, M, s.decay_rank, 1, st)));
            DenseCall c;
            c.epi  = kDenseBiasF32;
            c.bias = L.w0;
            TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_call(L.w2, lm.d_lora, lm.ldlora, lm.d_wdec, lm.ldmix, M, c, st)));
            TM_PROF(P_KV_STORE, TM_TRY(launch_delta_prep(lm.d_proj, lm.ldproj, L.c_k, L.c_a, lm.d_wdec, lm.ldmix, lm.d_aux, lm.ldmix, M, H, s.dim, st)));
        }
        for (int i = 0; i < nparts; ++i) {
            const LmPart&  P = parts[i];
            StateMixParams sp;
            sp.max_q_len = P.decode ? 1 : std::max(1, P.max_q_len);
            sp.nseq = P.nseq, sp.cu_q = P.cu_q, sp.k_len = P.k_len, sp.seq_slot = P.seq_slot, sp.slot0 = P.slot0, sp.active = P.active;
            sp.park_slot   = e->cfg.max_batch_size;
            sp.state       = lm.d_state;
            sp.slot_stride = lm.state_slot_floats, sp.layer_offset = L.state_offset;
            sp.heads = H, sp.dim = s.dim, sp.vdim = s.vdim;
            sp.proj = lm.d_proj + (size_t)P.row0 * lm.ldproj, sp.ld = lm.ldproj;
            sp.c_q = 0, sp.c_k = L.c_k, sp.c_v = L.c_v, sp.c_a = L.c_a;
            sp.decay_h = L.decay_d;
            sp.decay_w = lm.d_wdec + (size_t)P.row0 * lm.ldmix, sp.ld_w = lm.ldmix;
            sp.unit    = lm.d_aux + (size_t)P.row0 * lm.ldmix, sp.ld_u = lm.ldmix;
            sp.out     = lm.d_mixo + (size_t)P.row0 * lm.ldmix, sp.ldo = lm.ldmix;
            TM_PROF(P_ATTN, TM_TRY(launch_state_mix(sp, delta, st)));
        }
        TM_PROF(P_ATTN, TM_TRY(launch_gated_group_norm(lm.d_cat, lm.ldcat, lm.elem, lm.d_mixo, lm.ldmix, L.mix_norm, lm.d_proj + L.c_g, lm.ldproj, M,
                                                       delta ? H : 1, delta ? s.dim : L.n_att, m.norm_eps, st)));
    }
    TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.wo, lm.d_cat, lm.ldcat, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
    TM_PROF(P_RES_NORM, TM_TRY(launch_layernorm_add_f32(lm.d_res, lm.d_h1, lm.ldw, lm.elem, lm.d_y, L.norm1, L.norm1_b, m.norm_eps, M, W, st)));
    if (s.mlp == TM_MLP_NONE) {
        return 0;
    }
    if (s.mlp == TM_MLP_DENSE) {
        DenseCall c;
        c.epi     = s.act == TM_ACT_XIELU ? kDenseXielu : kDenseRelu2;
        c.act_par = L.act_par;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_call(L.up, lm.d_h1, lm.ldw, lm.d_ff, lm.ldff, M, c, st)));
        TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_linear(L.down, lm.d_ff, lm.ldff, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
    }
    else {
        const int k = s.top, E = s.experts;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_linear(L.router, lm.d_h1, lm.ldw, lm.d_proj, lm.ldproj, M, kDenseScaleF32, 1.f, st)));
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_topk_softmax(lm.d_topk_ids, lm.d_topk_w, lm.d_proj, lm.ldproj, M, E, k, s.router_scale, st)));
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_route(lm.d_offsets, lm.d_f2n, lm.d_en2f, lm.d_topk_ids, M, E, k, st)));
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_gather(lm.d_moe_x, lm.ldw, lm.d_h1, lm.ldw, lm.elem, lm.d_topk_w, lm.d_en2f, M, W, k, false, st)));
        int rows = M * k;
        if (L.shared_fused) {  // the shared expert: item E of the batched products over a copy of all rows behind the routed ones
            TM_HIP_CHECK(hipMemcpyAsync((char*)lm.d_moe_x + (size_t)rows * lm.ldw * lm.elem, lm.d_h1, (size_t)M * lm.ldw * lm.elem, hipMemcpyDeviceToDevice, st));
            TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_moe_extend_offsets(lm.d_offsets, E, M, st)));
            rows += M;
        }
        DenseCall c;
        c.epi         = kDenseRelu2;
        c.count       = E + (L.shared_fused ? 1 : 0);
        c.row_offsets = lm.d_offsets;
        TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_call(L.gu, lm.d_moe_x, lm.ldw, lm.d_ff, lm.ldff, rows, c, st)));
        c.epi = kDenseScaleF32;
        TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_call(L.down, lm.d_ff, lm.ldff, lm.d_moe_y, W, rows, c, st)));
        if (L.shared_fused) {
            TM_PROF(P_GEMM_DOWN, TM_TRY(launch_moe_combine_f32(lm.d_y, lm.d_moe_y, lm.d_topk_w, lm.d_en2f, nullptr, 0, nullptr, M, W, k, true, st, true,
                                                         lm.d_moe_y + (size_t)M * k * W)));
        }
        else if (s.shared_ff > 0) {  // the shared expert's result opens the sum, the routed experts join it
            TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_linear(L.sh_up, lm.d_h1, lm.ldw, lm.d_ff, lm.ldff, M, kDenseRelu2, 1.f, st)));
            TM_PROF(P_GEMM_DOWN, TM_TRY(launch_dense_linear(L.sh_down, lm.d_ff, lm.ldff, lm.d_y, W, M, kDenseScaleF32, 1.f, st)));
        }
        if (!L.shared_fused) {
            TM_PROF(P_GEMM_DOWN, TM_TRY(launch_moe_combine_f32(lm.d_y, lm.d_moe_y, lm.d_topk_w, lm.d_en2f, nullptr, 0, nullptr, M, W, k, true, st,
                                                         s.shared_ff <= 0)));
        }
    }
    TM_PROF(P_RES_NORM, TM_TRY(launch_layernorm_add_f32(lm.d_res, lm.d_h1, lm.ldw, lm.elem, lm.d_y, L.norm2, L.norm2_b, m.norm_eps, M, W, st)));
    return 0;
}

// the layer loop over M rows described by `parts`; leaves the residual stream in lm.d_res
static int layered_layers(tm_engine* e, const int* d_ids, int M, const LmPart* parts, int nparts)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    hipStream_t              st = e->stream;
    TM_REQUIRE(M >= 1 && M <= e->max_tokens, "forward: more rows than max_prefill_token_num");
    for (int i = 0; i < nparts; ++i) {
        const LmPart& P = parts[i];
        TM_TRY(launch_rows_prepare(lm.d_row_seq + P.row0, lm.d_row_pos + P.row0, P.cu_q, P.k_len, P.nseq, P.rows, st));
    }
    TM_PROF(P_EMBED, TM_TRY(launch_embedding_f32(lm.d_res, lm.embed, lm.elem, d_ids, M, m.width, m.vocab, st, m.embed_scale > 0.f ? m.embed_scale : 1.f)));
    if (m.loop_times > 0) {  // the embedding output is read again where a loop pass begins
        TM_PROF(P_EMBED, TM_TRY(launch_embedding_f32(lm.d_x0, lm.embed, lm.elem, d_ids, M, m.width, m.vocab, st)));
    }
    const int n_run = lm.debug_layers >= 0 ? std::min(lm.debug_layers, m.n_layers) : m.n_layers;
    for (int li = 0; li < n_run; ++li) {
        const LmLayer&       L = lm.layers[li];
        const tm_layer_spec& s = L.spec;
        if (s.loop_pass >= 0) {
            DenseCall c;
            c.epi  = kDenseBiasF32;
            c.bias = lm.loop_step + (size_t)s.loop_pass * m.width;
            TM_PROF(P_RES_NORM, TM_TRY(launch_concat2(lm.d_xx, lm.ld2w, lm.elem, lm.d_res, lm.d_x0, M, m.width, st)));
            TM_PROF(P_GEMM_O, TM_TRY(launch_dense_call(lm.loop_in, lm.d_xx, lm.ld2w, lm.d_res, m.width, M, c, st)));
        }
        if (L.post) {
            TM_TRY(post_layer(e, L, M, parts, nparts, li > 0 && lm.layers[li - 1].post));
            continue;
        }
        if (L.wide) {
            TM_TRY(wide_layer(e, L, M, parts, nparts));
            continue;
        }
        TM_PROF(P_RES_NORM, TM_TRY(launch_rmsnorm_f32(lm.d_h1, s.mlp ? lm.d_h2 : nullptr, lm.ldw, lm.elem, lm.d_res, nullptr, L.norm1, L.norm2,
                                                      m.norm_offset, m.norm_eps, M, m.width, st)));
        TM_PROF(P_GEMM_QKV, TM_TRY(launch_dense_linear(L.qkv, lm.d_h1, lm.ldw, lm.d_qkv, lm.ldqkv, M, kDenseStore, 1.f, st)));
        for (int i = 0; i < nparts; ++i) {
            const LmPart&     P = parts[i];
            GeneralAttnParams p = attn_params(e, L, P);
            TM_PROF(P_KV_STORE, TM_TRY(launch_kv_store_general(p.q, lm.ldqkv, L.n_q, L.n_q + L.n_k, p, st)));
            if (P.decode && lm.decode_splits > 1
                && general_attention_workspace_bytes(P.rows, s.heads, s.vdim, lm.decode_splits) <= lm.attn_ws_bytes) {
                p.splits     = lm.decode_splits;
                p.partial_o  = lm.d_attn_ws;
                p.partial_ml = lm.d_attn_ws + (size_t)P.rows * s.heads * p.splits * s.vdim;
            }
            TM_PROF(P_ATTN, TM_TRY(launch_general_attention(p, !P.decode, st)));
        }
        if (s.mlp) {
            TM_PROF(P_GEMM_GATE_UP, TM_TRY(launch_dense_linear(L.up, lm.d_h2, lm.ldw, (char*)lm.d_cat + (size_t)L.n_att * lm.elem, lm.ldcat, M,
                                                               kDenseRelu2, 1.f, st)));
        }
        TM_PROF(P_GEMM_O, TM_TRY(launch_dense_linear(L.out, lm.d_cat, lm.ldcat, lm.d_res, m.width, M, kDenseResidAdd, m.residual_mult, st)));
    }
    return 0;
}

// fp32 logits of `n` rows of the residual stream (rows == nullptr: rows 0 .. n-1) -> lm.d_logits_f32 [n][vocab]
static int layered_logits(tm_engine* e, const int* rows, int n)
{
    LayeredModel&            lm = *e->lm;
    const tm_layered_config& m  = lm.cfg;
    TM_REQUIRE(n <= lm.max_logit_rows, "internal: too many logits rows");
    if (m.norm_groups > 0) {
        TM_PROF(P_RES_NORM, TM_TRY(launch_group_rmsnorm_f32(lm.d_hn, lm.ldw, lm.elem, lm.d_res, rows, lm.final_norm, m.norm_groups, m.norm_eps, n, m.width,
                                                            e->stream)));
    }
    else if (m.final_layer_norm) {
        TM_PROF(P_RES_NORM, TM_TRY(launch_layernorm_f32(lm.d_hn, lm.ldw, lm.elem, lm.d_res, rows, lm.final_norm, lm.final_norm_b, m.norm_eps, n,
                                                        m.width, e->stream)));
    }
    else {
        TM_PROF(P_RES_NORM, TM_TRY(launch_rmsnorm_f32(lm.d_hn, nullptr, lm.ldw, lm.elem, lm.d_res, rows, lm.final_norm, nullptr, m.norm_offset,
                                                      m.norm_eps, n, m.width, e->stream)));
    }
    TM_PROF(P_LM_HEAD, TM_TRY(launch_dense_linear(lm.head, lm.d_hn, lm.ldw, lm.d_logits_f32, m.vocab, n, kDenseScaleF32, m.logit_scale, e->stream)));
    if (m.logit_softcap > 0.f) {
        TM_PROF(P_LM_HEAD, TM_TRY(launch_softcap_f32(lm.d_logits_f32, (size_t)n * m.vocab, m.logit_softcap, e->stream)));
    }
    return 0;
}

// logits of `n` sequences -> the engine's fp16 logits rows at the batch slots [slot, slot + n) -> logits processors + sampling
static int layered_head(tm_engine* e, const int* rows, int n, int slot, const int* ids_in, const int* cu_q, int ntok, const int* k_len,
                        const int* active)
{
    LayeredModel& lm = *e->lm;
    for (int r0 = 0; r0 < n; r0 += lm.max_logit_rows) {
        const int cnt = std::min(lm.max_logit_rows, n - r0);
        TM_TRY(layered_logits(e, rows + r0, cnt));
        TM_TRY(launch_f32_to_f16_rows(e->d_logits + (size_t)(slot + r0) * e->vocab_local, e->vocab_local, lm.d_logits_f32, cnt, lm.cfg.vocab,
                                      e->stream));
    }
    return sample_rows(e, n, slot, ids_in, cu_q, ntok, k_len, active);
}

// forward() of the engine for this family: the same batch description as every other model (engine_forward.hip)
int layered_forward(tm_engine* e, const int* d_ids, int M, int nseq, bool decode, int max_q_len, int max_k_len, int slot0, const MixedDecode* md)
{
    LayeredModel& lm = *e->lm;
    const int     nd = md ? md->rows : 0;
    TM_REQUIRE(!md || (!decode && nd > 0 && nd < M), "internal: mixed forward");
    LmPart parts[2];
    int    np = 0;
    if (md) {  // the decode rows of every batch slot first, on the decode state's own table
        parts[np++] = LmPart{0, nd, nd, md->cu_q, md->k_len, nullptr, md->block_ptrs, true, 1, 0, md->active};
    }
    // (the decode step of continuous batching runs every slot: those without a running sequence are placeholders)
    parts[np++] = LmPart{nd, M - nd, nseq, e->d_cu_q, e->d_k_len, nullptr, e->d_block_ptrs, decode, decode ? 1 : max_q_len, slot0,
                         decode && e->sched ? e->d_active : nullptr};
    TM_TRY(layered_layers(e, d_ids, M, parts, np));
    if (decode) {
        return layered_head(e, lm.d_iota, nseq, slot0, d_ids, nullptr, M, e->d_k_len, nullptr);
    }
    if (md) {
        TM_TRY(layered_head(e, lm.d_iota, nd, 0, d_ids, nullptr, nd, md->k_len, md->active));
    }
    return layered_head(e, e->d_rows, nseq, slot0, d_ids + nd, e->d_cu_q, M - nd, e->d_k_len, nullptr);  // d_rows: last row of every sequence
}

}  // namespace tmk

extern "C" {

int tm_engine_create_layered(tm_engine** out, const tm_engine_config* c, const tm_layered_config* m)
{
    TM_REQUIRE(out && c && m && m->layers, "null pointer");
    TM_REQUIRE(c->tp == 1 && c->rank == 0, "layer-list models run on one GPU (tp = 1)");
    TM_REQUIRE(c->quant_policy == 0, "layer-list models keep the cache in the activation type (quant_policy 0)");
    TM_REQUIRE(c->cache_block_seq_len == 64, "cache_block_seq_len must be 64");
    TM_REQUIRE(c->max_batch_size >= 1 && c->max_batch_size <= 1024 && c->session_len >= 1, "1 <= max_batch_size <= 1024, session_len >= 1");
    TM_REQUIRE(m->width >= 1 && m->vocab >= 1 && m->n_layers >= 1, "width, vocab, layers >= 1");
    TM_REQUIRE(m->dtype == TM_DTYPE_BF16 || m->dtype == TM_DTYPE_F32, "dtype: bf16 | f32");
    TM_REQUIRE(m->norm_eps > 0.f, "norm_eps > 0");
    for (int i = 0; i < m->n_layers; ++i) {
        const tm_layer_spec& s = m->layers[i];
        const std::string at = "layer " + std::to_string(i);
        TM_REQUIRE(s.mixer >= TM_MIXER_ATTENTION && s.mixer <= TM_MIXER_PARALLEL, at + ": unknown mixer");
        TM_REQUIRE(s.post_norm || (s.norm_groups == 0 && s.conv_taps == 0 && !s.diff_maps && !s.rot_pairs && s.yarn_factor == 0.f && s.mixer != TM_MIXER_PARALLEL),
                   at + ": group norms, convolved projections, differential attention, pairwise rotation and parallel mixers belong to post_norm blocks");
        if (s.post_norm && s.norm_groups > 0) {
            TM_REQUIRE(m->width % s.norm_groups == 0 && m->norm_groups > 0, at + ": the width is a multiple of norm_groups; the model's last norm is a group norm too");
            TM_REQUIRE(s.mixer == TM_MIXER_ATTENTION || s.mixer == TM_MIXER_PARALLEL, at + ": a block with group norms mixes by attention or by the parallel pair");
            TM_REQUIRE(s.weights_of < 0 && !s.one_norm && !s.resid_gate && s.loop_pass < 0 && !s.sink && !s.dist_bias && !s.out_gate && s.chunk == 0
                           && !s.qk_unit_norm && !s.v_unit_norm && s.qtemp_coef == 0.f && !s.qkv_bias && s.keep_first == 0,
                       at + ": a block with group norms takes none of the other block forms' switches");
            TM_REQUIRE(s.heads >= 1 && s.kv_heads >= 1 && s.heads % s.kv_heads == 0 && s.dim >= 1 && s.dim <= 256 && s.vdim >= 1 && s.vdim <= 256 && s.window >= 0,
                       at + ": heads % kv_heads, 1 <= dim, vdim <= 256, window >= 0");
            TM_REQUIRE(s.conv_taps >= 0 && s.conv_taps <= 16, at + ": at most 16 taps");
            TM_REQUIRE(s.mlp == TM_MLP_NONE || (s.mlp == TM_MLP_GATED && s.ff >= 1 && s.act >= TM_ACT_RELU2 && s.act <= TM_ACT_SILU), at + ": gated feed-forward");
            if (s.mixer == TM_MIXER_ATTENTION) {
                TM_REQUIRE(s.rot_dims >= 0 && s.rot_dims % 2 == 0 && s.rot_dims <= s.dim && s.rot_base > 0.f && s.rot_scale > 0.f,
                           at + ": rot_dims even and <= dim, rot_base, rot_scale > 0");
                TM_REQUIRE(s.yarn_factor == 0.f || (s.yarn_factor > 0.f && s.yarn_original > 0.f && s.yarn_fast > 0.f && s.yarn_slow > 0.f && s.rot_base != 1.f),
                           at + ": frequency scaling: factor, original, fast, slow > 0");
            }
            else {
                TM_REQUIRE(s.vdim == s.dim && s.kv_heads * s.dim <= 1024 && s.heads * s.dim <= 12288 && s.dist_buckets >= 2 && s.dist_max > s.dist_buckets / 2
                               && !s.diff_maps && s.conv_taps == 0 && s.rot_dims == 0 && s.softcap <= 0.f,
                           at + ": left mixer: vdim = dim, kv_heads * dim <= 1024, dist_buckets >= 2, dist_max > dist_buckets / 2, no maps / convolution / rotation / cap");
                TM_REQUIRE(s.r_heads >= 1 && s.r_kv_heads >= 1 && s.r_heads % s.r_kv_heads == 0 && s.r_dim >= 1 && s.r_dim <= 256 && s.r_vdim >= 1
                               && s.r_vdim <= 1024 && s.r_conv >= 1 && s.r_conv <= 16 && s.a_rank >= 1 && s.g_rank >= 1,
                           at + ": right mixer: r_heads % r_kv_heads, 1 <= r_dim <= 256, 1 <= r_vdim <= 1024, 1 <= r_conv <= 16, a_rank, g_rank >= 1");
            }
            continue;
        }
        TM_REQUIRE(s.post_norm || (s.mixer != TM_MIXER_LIGHTNING && s.mixer != TM_MIXER_DELTA && !s.qkv_bias && !s.qk_norm_w && s.window == 0
                                   && !s.expert_plain && !s.router_softmax && s.shared_ff == 0 && s.act != TM_ACT_XIELU),
                   at + ": state mixers, projection biases, weighted query / key norms, windows, plain experts and xIELU belong to post_norm blocks");
        TM_REQUIRE(s.window >= 0 && s.keep_first >= 0, at + ": window, keep_first >= 0");
        TM_REQUIRE(s.heads >= 1 && s.kv_heads >= 1 && s.heads % s.kv_heads == 0, at + ": heads % kv_heads");
        TM_REQUIRE(s.dim >= 1 && s.dim <= 256 && s.vdim >= 1 && s.vdim <= 256, at + ": 1 <= dim, vdim <= 256");
        TM_REQUIRE(s.chunk >= 0 && s.loop_pass < m->loop_times, at + ": chunk >= 0, loop_pass < loop_times");
        if (s.post_norm) {
            TM_REQUIRE(s.weights_of < 0 && !s.one_norm && !s.resid_gate && s.loop_pass < 0 && !s.sink && !s.dist_bias && !s.out_gate && s.chunk == 0
                           && !s.qk_unit_norm && !s.v_unit_norm && s.softcap <= 0.f && s.qtemp_coef == 0.f && s.mixer != TM_MIXER_LATENT,
                       at + ": a post_norm block takes none of the other block forms' switches");
            TM_REQUIRE(m->final_layer_norm && m->norm_groups == 0, at + ": post_norm blocks with layer norms end in a final layer norm");
            TM_REQUIRE(s.mixer != TM_MIXER_PARALLEL && s.conv_taps == 0 && !s.diff_maps && !s.rot_pairs && s.yarn_factor == 0.f,
                       at + ": the parallel pair, convolved projections, differential attention and pairwise rotation need norm_groups > 0");
            if (s.mixer == TM_MIXER_ATTENTION) {
                TM_REQUIRE(s.rot_dims >= 0 && s.rot_dims % 2 == 0 && s.rot_dims <= s.dim && s.rot_base > 0.f && s.rot_scale > 0.f,
                           at + ": rot_dims even and <= dim, rot_base, rot_scale > 0");
            }
            else {
                TM_REQUIRE(s.kv_heads == s.heads, at + ": a state mixer has one key / value head per query head");
                TM_REQUIRE(s.mixer != TM_MIXER_LIGHTNING || s.decay, at + ": lightning needs one decay per head");
                TM_REQUIRE(s.mixer != TM_MIXER_DELTA || (s.vdim == s.dim && s.decay_rank >= 1), at + ": delta rule: vdim = dim, decay_rank >= 1");
            }
            TM_REQUIRE(s.mlp == TM_MLP_NONE || (s.mlp == TM_MLP_DENSE && s.ff >= 1 && (s.act == TM_ACT_XIELU || s.act == TM_ACT_RELU2))
                           || (s.mlp == TM_MLP_MOE && s.ff >= 1 && s.expert_plain && s.router_softmax && s.act == TM_ACT_RELU2 && s.experts >= 1
                               && s.experts <= 1024 && s.top >= 1 && s.top <= s.experts && s.shared_ff >= 0),
                       at + ": feed-forward of a post_norm block: dense (xIELU | relu^2) or soft-max-routed plain relu^2 experts");
        }
        else if (layer_wide(s)) {
            TM_REQUIRE(s.one_norm, at + ": gates, per-head norms, latent attention and gated feed-forwards read ONE norm of the stream (one_norm)");
            TM_REQUIRE(s.mlp == TM_MLP_NONE || ((s.mlp == TM_MLP_GATED || s.mlp == TM_MLP_MOE) && s.ff >= 1 && s.act >= TM_ACT_RELU2 && s.act <= TM_ACT_SILU),
                       at + ": feed-forward");
            TM_REQUIRE(s.mlp != TM_MLP_MOE || (s.experts >= 1 && s.experts <= 1024 && s.top >= 1 && s.top <= s.experts), at + ": 1 <= top <= experts <= 1024");
            if (s.mixer == TM_MIXER_LATENT) {
                TM_REQUIRE(s.rot_dims >= 0 && s.rot_dims <= s.rot_dim && s.rot_dims % 2 == 0, at + ": rot_dims even, <= rot_dim");
                TM_REQUIRE(s.kv_heads == 1 && s.kv_rank >= 1 && s.rot_dim >= 0 && s.rot_dim % 2 == 0 && s.kv_rank + s.rot_dim <= 1024 && s.rot_base > 0.f,
                           at + ": latent attention: kv_heads 1, kv_rank >= 1, rot_dim even, kv_rank + rot_dim <= 1024");
                TM_REQUIRE(!s.qk_unit_norm && !s.v_unit_norm && !s.out_gate, at + ": latent attention has no per-head unit norms and no output gate");
            }
        }
        else {
            TM_REQUIRE(s.mlp == TM_MLP_NONE || (s.mlp == TM_MLP_DENSE && s.ff >= 1 && s.act == TM_ACT_RELU2), at + ": feed-forward");
        }
        TM_REQUIRE(s.qtemp_coef == 0.f || s.qtemp_every > 0.f, "layer " + std::to_string(i) + ": query temperature period");
        TM_REQUIRE(s.weights_of < 0 || (s.weights_of < m->n_layers && s.weights_of != i && m->layers[s.weights_of].weights_of < 0),
                   "layer " + std::to_string(i) + ": weights_of must name a layer with tensors of its own");
        if (s.weights_of >= 0) {
            const tm_layer_spec& o = m->layers[s.weights_of];
            TM_REQUIRE(o.heads == s.heads && o.kv_heads == s.kv_heads && o.dim == s.dim && o.vdim == s.vdim && o.mlp == s.mlp && o.ff == s.ff
                           && o.sink == s.sink,
                       "layer " + std::to_string(i) + ": sizes differ from the layer whose weights it uses");
            TM_REQUIRE(layer_wide(o) == layer_wide(s) && o.mixer == s.mixer && o.kv_rank == s.kv_rank && o.rot_dim == s.rot_dim && o.experts == s.experts
                           && o.resid_gate == s.resid_gate && o.out_gate == s.out_gate && o.dist_bias == s.dist_bias,
                       "layer " + std::to_string(i) + ": form differs from the layer whose weights it uses");
        }
    }
    TM_HIP_CHECK(hipSetDevice(c->device));
    auto* e = new tm_engine();
    e->cfg  = *c;
    memset(&e->cfg.model, 0, sizeof(e->cfg.model));
    e->cfg.model.hidden = m->width;
    e->cfg.model.layers = m->n_layers;
    e->cfg.model.vocab  = m->vocab;
    e->hidden           = m->width;
    e->vocab_local      = (m->vocab + 7) / 8 * 8;  // fp16 logits rows of the sampler: 16-byte aligned, pad columns never win
    e->q_heads = e->kv_heads = 1;                  // (the decode-split heuristic of the fixed-head-size kernels reads them; unused here)
    e->mixed_steps_on   = !(getenv("TM_MIXED_STEP") && !atoi(getenv("TM_MIXED_STEP")));
    TM_HIP_CHECK(hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking));
    e->lm.reset(new LayeredModel());
    LayeredModel& lm = *e->lm;
    lm.cfg           = *m;
    lm.cfg.layers    = nullptr;
    lm.elem          = m->dtype == TM_DTYPE_F32 ? 4 : 2;
    lm.layers.resize(m->n_layers);
    const int64_t W = m->width;
    for (int i = 0; i < m->n_layers; ++i) {
        LmLayer& L = lm.layers[i];
        L.spec     = m->layers[i];
        L.src      = L.spec.weights_of >= 0 ? L.spec.weights_of : i;
        L.n_q      = L.spec.heads * L.spec.dim;
        L.n_k      = L.spec.kv_heads * L.spec.dim;
        L.n_v      = L.spec.kv_heads * L.spec.vdim;
        L.n_att    = L.spec.heads * L.spec.vdim;
        L.a_dim = L.spec.dim, L.a_vdim = L.spec.vdim, L.a_kv = L.spec.kv_heads, L.a_heads = L.spec.heads;
        L.post = L.spec.post_norm != 0;
        L.has_state = L.spec.mixer == TM_MIXER_LIGHTNING || L.spec.mixer == TM_MIXER_DELTA || L.spec.mixer == TM_MIXER_PARALLEL;
        L.has_cache = L.spec.mixer != TM_MIXER_LIGHTNING && L.spec.mixer != TM_MIXER_DELTA;
        L.wide = !L.post && layer_wide(L.spec);
        auto slot = [&](const std::string& name, int64_t rows, int64_t cols) {
            e->slots[name].bytes = rows * cols * 2;
            lm.fan_in[name]      = (int)cols;
        };
        if (L.post && L.spec.norm_groups > 0) {
            const tm_layer_spec& s = L.spec;
            const int            H = s.heads, G = s.kv_heads, d = s.dim, dv = s.vdim;
            lm.has_post = true;
            slot(lname(i, "norm1"), 1, W);
            if (s.mixer == TM_MIXER_ATTENTION) {
                const int maps = s.diff_maps ? 2 : 1;
                L.n_q = H * maps * d, L.n_k = G * maps * d, L.n_v = G * dv, L.n_att = H * dv;
                L.a_heads = H * maps, L.a_kv = G * maps;
                if (maps > 1) {  // both maps of a head read the head's one value head
                    L.a_kh = G * maps, L.a_vh = G;
                }
                L.c_k = L.n_q, L.c_v = L.c_k + L.n_k, L.c_g = L.c_end = L.c_v + L.n_v;
                slot(lname(i, "mix.q"), L.n_q, W);
                slot(lname(i, "mix.k"), L.n_k, W);
                slot(lname(i, "mix.v"), L.n_v, W);
                slot(lname(i, "mix.o"), W, L.n_att);
                if (s.qk_norm_w) {
                    slot(lname(i, "mix.q.norm"), 1, d);
                    slot(lname(i, "mix.k.norm"), 1, d);
                }
                if (s.conv_taps > 0) {
                    L.conv_col = 0, L.conv_ch = L.c_end, L.conv_taps = s.conv_taps, L.conv_act = 0;
                    slot(lname(i, "mix.q.conv"), L.n_q, s.conv_taps);
                    slot(lname(i, "mix.k.conv"), L.n_k, s.conv_taps);
                    slot(lname(i, "mix.v.conv"), L.n_v, s.conv_taps);
                }
                if (s.diff_maps) {
                    for (const char* t : {"mix.lq1", "mix.lk1", "mix.lq2", "mix.lk2"}) {
                        slot(lname(i, t), 1, d);
                    }
                }
            }
            else {
                const int Hr = s.r_heads, Gr = s.r_kv_heads, dr = s.r_dim, dvr = s.r_vdim;
                // left: one wide key [G dim] shared by all heads (the head mixing lives in the queries), a value head per group
                L.n_q = H * d, L.n_k = G * d, L.n_v = G * dv, L.n_att = H * dv;
                L.a_heads = H, L.a_kv = G, L.a_kh = 1, L.a_vh = G, L.a_dim = G * d, L.a_vdim = dv;
                L.r_nqk = Gr * dr, L.r_nv = Hr * dvr;
                L.c_k = L.n_q, L.c_g = L.c_k + L.n_k, L.c_rq = L.c_g + L.n_att, L.c_rk = L.c_rq + L.r_nqk, L.c_rv = L.c_rk + L.r_nqk;
                L.c_b = L.c_rv + L.r_nv, L.c_a1 = L.c_b + Hr, L.lora_g1 = (s.a_rank + 31) / 32 * 32, L.c_g1 = L.c_a1 + L.lora_g1;
                L.c_end = L.c_g1 + s.g_rank;
                L.conv_col = L.c_rq, L.conv_ch = 2 * L.r_nqk + L.r_nv, L.conv_taps = s.r_conv, L.conv_act = 1;
                L.c_xq = L.conv_ch, L.c_xk = L.c_xq + Hr * dr;
                slot(lname(i, "mix.left.q"), L.n_q, W);
                slot(lname(i, "mix.left.k"), L.n_k, W);
                slot(lname(i, "mix.left.q.norm"), 1, L.n_q);
                slot(lname(i, "mix.left.k.norm"), 1, L.n_k);
                slot(lname(i, "mix.left.rel"), s.dist_buckets, H);
                slot(lname(i, "mix.left.talk"), H, H);
                slot(lname(i, "mix.left.g"), L.n_att, W);
                slot(lname(i, "mix.left.o"), W, L.n_att);
                slot(lname(i, "mix.left.out"), 1, W);
                slot(lname(i, "mix.right.q"), L.r_nqk, W);
                slot(lname(i, "mix.right.k"), L.r_nqk, W);
                slot(lname(i, "mix.right.v"), L.r_nv, W);
                slot(lname(i, "mix.right.q.conv"), L.r_nqk, s.r_conv);
                slot(lname(i, "mix.right.k.conv"), L.r_nqk, s.r_conv);
                slot(lname(i, "mix.right.v.conv"), L.r_nv, s.r_conv);
                slot(lname(i, "mix.right.b"), Hr, W);
                slot(lname(i, "mix.right.A_log"), 1, Hr);
                slot(lname(i, "mix.right.norm"), 1, dvr);
                slot(lname(i, "mix.right.a1"), s.a_rank, W);
                slot(lname(i, "mix.right.a2"), (int64_t)Hr * dr, s.a_rank);
                slot(lname(i, "mix.right.dt_bias"), 1, (int64_t)Hr * dr);
                slot(lname(i, "mix.right.g1"), s.g_rank, W);
                slot(lname(i, "mix.right.g2"), L.r_nv, s.g_rank);
                slot(lname(i, "mix.right.o"), W, L.r_nv);
                slot(lname(i, "mix.right.out"), 1, W);
            }
            if (s.mlp) {
                slot(lname(i, "norm2"), 1, W);
                slot(lname(i, "mlp.gate"), s.ff, W);
                slot(lname(i, "mlp.up"), s.ff, W);
                slot(lname(i, "mlp.down"), W, s.ff);
            }
            continue;
        }
        if (L.post) {
            const tm_layer_spec& s = L.spec;
            const int            H = s.heads;
            lm.has_post = true;
            L.c_k = L.n_q, L.c_v = L.c_k + L.n_k, L.c_g = L.c_v + L.n_v, L.c_end = L.c_g;
            L.shared_fused = s.mlp == TM_MLP_MOE && s.shared_ff > 0 && s.shared_ff <= s.ff;
            slot(lname(i, "norm1"), 1, W);
            slot(lname(i, "norm1.b"), 1, W);
            slot(lname(i, s.mixer == TM_MIXER_DELTA ? "mix.r" : "mix.q"), L.n_q, W);
            slot(lname(i, "mix.k"), L.n_k, W);
            slot(lname(i, "mix.v"), L.n_v, W);
            slot(lname(i, "mix.o"), W, L.n_att);
            if (s.mixer == TM_MIXER_ATTENTION) {
                if (s.qkv_bias) {
                    slot(lname(i, "mix.q.b"), 1, L.n_q);
                    slot(lname(i, "mix.k.b"), 1, L.n_k);
                    slot(lname(i, "mix.v.b"), 1, L.n_v);
                }
                if (s.qk_norm_w) {
                    slot(lname(i, "mix.q.norm"), 1, s.dim);
                    slot(lname(i, "mix.k.norm"), 1, s.dim);
                }
            }
            else {
                L.c_end = L.c_g + L.n_att;
                slot(lname(i, "mix.g"), L.n_att, W);
                slot(lname(i, "mix.norm"), 1, L.n_att);
                if (s.mixer == TM_MIXER_LIGHTNING) {
                    L.decay_h.assign(s.decay, s.decay + H);
                    L.spec.decay = nullptr;
                }
                else {
                    L.c_a = L.c_end, L.c_w1 = L.c_a + L.n_q, L.c_end = L.c_w1 + s.decay_rank;
                    slot(lname(i, "mix.a"), L.n_q, W);
                    slot(lname(i, "mix.a.b"), 1, L.n_q);
                    slot(lname(i, "mix.w1"), s.decay_rank, W);
                    slot(lname(i, "mix.w2"), L.n_q, s.decay_rank);
                    slot(lname(i, "mix.w0"), 1, L.n_q);
                }
            }
            if (s.mlp) {
                slot(lname(i, "norm2"), 1, W);
                slot(lname(i, "norm2.b"), 1, W);
            }
            if (s.mlp == TM_MLP_DENSE) {
                slot(lname(i, "mlp.up"), s.ff, W);
                slot(lname(i, "mlp.down"), W, s.ff);
                if (s.act == TM_ACT_XIELU) {
                    slot(lname(i, "mlp.act"), 1, 2);
                }
            }
            else if (s.mlp == TM_MLP_MOE) {
                slot(lname(i, "mlp.router"), s.experts, W);
                for (int x = 0; x < s.experts; ++x) {
                    const std::string ex = "mlp.e" + std::to_string(x) + ".";
                    slot(lname(i, (ex + "up").c_str()), s.ff, W);
                    slot(lname(i, (ex + "down").c_str()), W, s.ff);
                }
                if (s.shared_ff > 0) {
                    slot(lname(i, "mlp.shared.up"), s.shared_ff, W);
                    slot(lname(i, "mlp.shared.down"), W, s.shared_ff);
                }
            }
            continue;
        }
        if (L.wide) {
            const tm_layer_spec& s = L.spec;
            const int            H = s.heads;
            int                  next;
            if (s.mixer == TM_MIXER_LATENT) {  // the cache holds one key head [kv_rank | rot_dim] and the latent vector as its value
                L.a_dim = s.kv_rank + s.rot_dim, L.a_vdim = s.kv_rank, L.a_kv = 1;
                L.n_q = H * (s.dim + s.rot_dim), L.n_k = L.a_dim, L.n_v = L.a_vdim;
                L.plain_stride = (s.dim + 31) / 32 * 32, L.lat_stride = (s.kv_rank + 31) / 32 * 32;
                L.c_k = L.n_q;
                next  = L.c_k + s.kv_rank + s.rot_dim;
            }
            else {
                L.c_k = L.n_q, L.c_v = L.c_k + L.n_k, L.c_g = L.c_v + L.n_v;
                next  = L.c_g + (s.out_gate ? H : 0);
            }
            L.c_rg1 = next, next += s.resid_gate ? (int)W : 0;
            L.c_rg2 = next, next += s.resid_gate && s.mlp ? (int)W : 0;
            L.c_router = next;
            if (L.src != i) {
                continue;
            }
            slot(lname(i, "norm1"), 1, W);
            slot(lname(i, "mix.q"), L.n_q, W);
            slot(lname(i, "mix.o"), W, L.n_att);
            if (s.mixer == TM_MIXER_LATENT) {
                slot(lname(i, "mix.dkv"), s.kv_rank + s.rot_dim, W);
                slot(lname(i, "mix.dkv.norm"), 1, s.kv_rank);
                slot(lname(i, "mix.uk"), (int64_t)H * s.dim, s.kv_rank);
                slot(lname(i, "mix.uv"), (int64_t)H * s.vdim, s.kv_rank);
            }
            else {
                slot(lname(i, "mix.k"), L.n_k, W);
                slot(lname(i, "mix.v"), L.n_v, W);
                if (s.out_gate) {
                    slot(lname(i, "mix.g"), H, W);
                }
            }
            if (s.dist_bias) {
                slot(lname(i, "mix.r1"), 1, H);
                slot(lname(i, "mix.r2"), 1, H);
            }
            if (s.sink) {
                slot(lname(i, "mix.sink"), 1, H);
            }
            if (s.resid_gate) {
                slot(lname(i, "rg1"), W, W);
                slot(lname(i, "rg1.b"), 1, W);
                if (s.mlp) {
                    slot(lname(i, "rg2"), W, W);
                    slot(lname(i, "rg2.b"), 1, W);
                }
            }
            if (s.mlp == TM_MLP_GATED) {
                slot(lname(i, "mlp.gate"), s.ff, W);
                slot(lname(i, "mlp.up"), s.ff, W);
                slot(lname(i, "mlp.down"), W, s.ff);
            }
            else if (s.mlp == TM_MLP_MOE) {
                slot(lname(i, "mlp.router"), s.experts, W);
                for (int x = 0; x < s.experts; ++x) {
                    const std::string ex = "mlp.e" + std::to_string(x) + ".";
                    slot(lname(i, (ex + "gate").c_str()), s.ff, W);
                    slot(lname(i, (ex + "up").c_str()), s.ff, W);
                    slot(lname(i, (ex + "down").c_str()), W, s.ff);
                }
            }
            continue;
        }
        if (L.src != i) {
            continue;
        }
        e->slots[lname(i, "norm1")].bytes = W * 2;
        e->slots[lname(i, "mix.q")].bytes = W * L.n_q * 2;
        e->slots[lname(i, "mix.k")].bytes = W * L.n_k * 2;
        e->slots[lname(i, "mix.v")].bytes = W * L.n_v * 2;
        e->slots[lname(i, "mix.o")].bytes = W * L.n_att * 2;
        if (L.spec.sink) {
            e->slots[lname(i, "mix.sink")].bytes = (int64_t)L.spec.heads * 2;
        }
        if (L.spec.mlp) {
            e->slots[lname(i, "norm2")].bytes    = W * 2;
            e->slots[lname(i, "mlp.up")].bytes   = W * L.spec.ff * 2;
            e->slots[lname(i, "mlp.down")].bytes = W * L.spec.ff * 2;
        }
    }
    if (m->loop_times > 0) {
        e->slots["loop.in"].bytes   = W * 2 * W * 2;
        lm.fan_in["loop.in"]        = (int)(2 * W);
        e->slots["loop.step"].bytes = (int64_t)m->loop_times * W * 2;
    }
    e->slots["embed"].bytes      = W * m->vocab * 2;
    e->slots["final.norm"].bytes = W * 2;
    if (m->final_layer_norm && m->norm_groups == 0) {
        e->slots["final.norm.b"].bytes = W * 2;
    }
    e->slots["head"].bytes       = W * m->vocab * 2;
    *out = e;
    return 0;
}

int tm_engine_debug_stop_after(tm_engine* e, int layers)
{
    TM_REQUIRE(e && e->lm, "layer-list engine");
    e->lm->debug_layers = layers;
    return 0;
}

int tm_engine_session_open(tm_engine* e, int64_t* session)
{
    TM_REQUIRE(e && session, "null pointer");
    TM_REQUIRE(e->lm, "sessions need a layer-list model");
    if (e->loop_on.load()) {
        set_last_error("the engine thread is running (tm_engine_serve_stop first)");
        return TM_CONFLICT;
    }
    ApiLock lk(e);
    TM_TRY(cb_enter(e));
    if (e->sched->n_active() > e->sched->n_sessions() || e->sched->n_waiting() > 0) {
        set_last_error("queued / running requests exist: sessions and tm_engine_submit do not share a scheduler session");
        return TM_CONFLICT;
    }
    if (e->sched->open_session(session)) {
        set_last_error("no free batch slot");
        return TM_CONFLICT;
    }
    e->lm->sess_len[*session] = 0;
    return 0;
}

int tm_engine_session_close(tm_engine* e, int64_t session)
{
    TM_REQUIRE(e && e->lm && e->sched, "no open session");
    ApiLock lk(e);
    TM_HIP_CHECK(hipStreamSynchronize(e->stream));
    TM_REQUIRE(e->sched->close_session(session) == 0, "unknown session");
    e->lm->sess_len.erase(session);
    return 0;
}

int tm_engine_step_tokens(tm_engine* e, const tm_step_entry* entries, int n_entries, float* host_logits)
{
    TM_REQUIRE(e && entries && n_entries >= 1, "null pointer / no entries");
    TM_REQUIRE(e->lm && e->sched, "no open session");
    ApiLock       lk(e);
    LayeredModel& lm = *e->lm;
    TM_HIP_CHECK(hipSetDevice(e->cfg.device));
    TM_REQUIRE(n_entries <= e->cfg.max_batch_size, "more entries than batch slots");
    // decoded tokens (one row) first, portions after them: two parts of one forward, each on its kind of attention kernel
    std::vector<int> order;
    for (int pass = 0; pass < 2; ++pass) {
        for (int i = 0; i < n_entries; ++i) {
            TM_REQUIRE(entries[i].n_tokens >= 1 && entries[i].tokens, "entry without tokens");
            if ((entries[i].n_tokens == 1) == (pass == 0)) {
                order.push_back(i);
            }
        }
    }
    int need = 0, total = 0, n_dec = 0;
    for (int i = 0; i < n_entries; ++i) {
        const tm_step_entry& en = entries[i];
        auto                 it = lm.sess_len.find(en.session);
        TM_REQUIRE(it != lm.sess_len.end(), "unknown session");
        for (int j = 0; j < i; ++j) {
            TM_REQUIRE(entries[j].session != en.session, "a session appears twice in one step");
        }
        const int nb = e->sched->grow_need(en.session, it->second + en.n_tokens);
        if (nb < 0) {
            set_last_error("session exceeds session_len");
            return TM_TOO_LONG;
        }
        need += nb;
        total += en.n_tokens;
        n_dec += en.n_tokens == 1;
        for (int w = 0; w < en.n_want; ++w) {
            TM_REQUIRE(en.want && en.want[w] >= 0 && en.want[w] < en.n_tokens, "want: index outside the entry's tokens");
        }
    }
    TM_REQUIRE(total <= e->max_tokens, "step brings more tokens than max_prefill_token_num");
    if (need > e->sched->n_free_blocks()) {
        set_last_error("out of KV cache blocks");
        return TM_OOM;
    }
    std::vector<int> ids, cu_q{0}, k_len, slots, want;
    std::vector<int> want_of(n_entries + 1, 0);  // logits rows are returned in ENTRY order: remember where each entry's rows start
    int              max_q = 1;
    std::vector<std::vector<int>> want_rows(n_entries);
    for (int oi : order) {
        const tm_step_entry& en  = entries[oi];
        int&                 len = lm.sess_len[en.session];
        const SchedRequest*  r   = e->sched->find(en.session);
        const size_t         had = r->blocks.size();
        TM_REQUIRE(e->sched->grow(en.session, len + en.n_tokens), "internal: block accounting");
        if (r->blocks.size() > had) {  // new blocks join the session's row of the block table
            std::vector<uint64_t> ptrs;
            for (size_t q = had; q < r->blocks.size(); ++q) {
                ptrs.push_back((uint64_t)(e->pool + (int64_t)r->blocks[q] * e->block_bytes));
            }
            TM_HIP_CHECK(hipMemcpyAsync(e->d_block_ptrs + (size_t)r->slot * e->max_blocks_per_seq + had, ptrs.data(), ptrs.size() * 8,
                                        hipMemcpyHostToDevice, e->stream));
            TM_HIP_CHECK(hipStreamSynchronize(e->stream));
        }
        for (int w = 0; w < en.n_want; ++w) {
            want_rows[oi].push_back((int)ids.size() + en.want[w]);
        }
        ids.insert(ids.end(), en.tokens, en.tokens + en.n_tokens);
        cu_q.push_back((int)ids.size());
        len += en.n_tokens;
        k_len.push_back(len);
        slots.push_back(r->slot);
        max_q = std::max(max_q, en.n_tokens);
    }
    for (int i = 0; i < n_entries; ++i) {
        want.insert(want.end(), want_rows[i].begin(), want_rows[i].end());
    }
    hipStream_t st = e->stream;
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_ids, ids.data(), ids.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_cu_q, cu_q.data(), cu_q.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_step_k_len, k_len.data(), k_len.size() * 4, hipMemcpyHostToDevice, st));
    TM_HIP_CHECK(hipMemcpyAsync(lm.d_seq_slot, slots.data(), slots.size() * 4, hipMemcpyHostToDevice, st));
    if (!want.empty()) {
        TM_HIP_CHECK(hipMemcpyAsync(lm.d_want, want.data(), want.size() * 4, hipMemcpyHostToDevice, st));
    }
    LmPart parts[2];
    int    np = 0;
    if (n_dec > 0) {
        parts[np++] = LmPart{0, n_dec, n_dec, lm.d_step_cu_q, lm.d_step_k_len, lm.d_seq_slot, e->d_block_ptrs, true, 1};
    }
    if (n_dec < n_entries) {
        // the portions' description starts at entry n_dec: cu_q values count from row 0 of the forward, the part's rows from n_dec
        parts[np++] = LmPart{n_dec, total - n_dec, n_entries - n_dec, lm.d_step_cu_q + n_dec, lm.d_step_k_len + n_dec, lm.d_seq_slot + n_dec,
                             e->d_block_ptrs, false, max_q};
    }
    int rc = layered_layers(e, lm.d_step_ids, total, parts, np);
    const int V = lm.cfg.vocab;
    for (size_t r0 = 0; rc == 0 && r0 < want.size(); r0 += lm.max_logit_rows) {
        const int cnt = (int)std::min<size_t>(lm.max_logit_rows, want.size() - r0);
        rc            = layered_logits(e, lm.d_want + r0, cnt);
        if (rc == 0) {
            TM_REQUIRE(host_logits, "host_logits is null but logits are wanted");
            TM_HIP_CHECK(hipMemcpyAsync(host_logits + r0 * V, lm.d_logits_f32, (size_t)cnt * V * 4, hipMemcpyDeviceToHost, st));
            TM_HIP_CHECK(hipStreamSynchronize(st));
        }
    }
    TM_HIP_CHECK(hipStreamSynchronize(st));  // the host vectors above are pageable
    return rc;
}

}  // extern "C"
