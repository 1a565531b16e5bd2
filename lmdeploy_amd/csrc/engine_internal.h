// Internal header of the engine translation units (engine.hip: configuration, weights, start / destroy; engine_forward.hip: the
// forward pass, static-batch prefill / decode, hipGraph capture; engine_comm.hip: tensor-parallel collectives and communicator set-up;
// engine_tune.hip: the measured GEMM dispatch; engine_serve.hip: continuous batching and the engine thread).  Not part of the C-ABI.
#pragma once
#include "../../include/tm_mi355x.h"
#include "scheduler.h"
#include "tm_common.h"
#include "tm_kernels.h"
#include <algorithm>
#include <atomic>
#include <cmath>
#include <condition_variable>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <mutex>
#include <rccl/rccl.h>
#include <thread>
#include <chrono>
#include <string>
#include <tuple>
#include <vector>


namespace tmk {

int build_rope_table(half_t* out, int max_pos, int dim, float base, int type, float factor, float low, float high,
                     int orig_max_pos);

#define TM_NCCL_CHECK(expr)                                                                        \
    do {                                                                                           \
        ncclResult_t _r = (expr);                                                                  \
        if (_r != ncclSuccess) {                                                                   \
            ::tmk::set_last_error(std::string(#expr) + ": " + ncclGetErrorString(_r));             \
            return 5;                                                                              \
        }                                                                                          \
    } while (0)

#define TM_TRY(expr)                                                                               \
    do {                                                                                           \
        int _rc = (expr);                                                                          \
        if (_rc) {                                                                                 \
            return _rc;                                                                            \
        }                                                                                          \
    } while (0)

// ---------------------------------------------------------------------------------------------
struct Slot {
    void*   dev   = nullptr;  // staging (boundary layout) -- freed by process_weights for linears
    int64_t bytes = 0;
    bool    filled = false;
};

struct LinearSlots {
    LinearWeight w;
    std::string  prefix;
};

struct Layer {
    LinearSlots qkv, wo, w13, w2;
    half_t*     attn_norm = nullptr;
    half_t*     ffn_norm  = nullptr;
    // mixture of experts: the dense w13 / w2 are unused; gate slot + per-expert slots feed `moe`
    bool                     is_moe = false;
    std::vector<LinearSlots> ex13, ex2;
    MoeBlock                 moe;
};

// ---- layer-list model family (engine_layered.hip) ------------------------------------------------------------------------------
// A model is a list of residual blocks, each naming its mixer, the mixer's sizes and constants, and its feed-forward; a layer may run on
// another layer's weights with a cache of its own.  The residual stream is fp32; activations and the cache are bf16 or fp32 (dtype).
struct LmLayer {
    tm_layer_spec spec{};
    int           src = 0;           // the layer whose weights this one runs on (itself unless spec.weights_of >= 0)
    DenseWeight   qkv, up, out;      // [q | k | v] along N; up; [o | down] along K.  Owned by layer `src`
    float *       norm1 = nullptr, *norm2 = nullptr, *sink = nullptr;
    int           n_q = 0, n_k = 0, n_v = 0, n_att = 0;  // heads * dim, kv_heads * dim, kv_heads * vdim, heads * vdim
    int64_t       kv_offset = 0, v_offset = 0;           // this layer's keys inside a cache block; its values behind the keys
    // blocks whose projections leave the fused product in fp32 (per-head norms, rotation, gates and routers read them): `qkv` then holds
    // every projection of the block's input h side by side, columns
    //   attention: [q | k | v | out gate | residual gate 1 | residual gate 2 | router]     latent: [q | dkv | residual gate 1 | 2 | router]
    bool          wide = false;
    int           a_dim = 0, a_vdim = 0, a_kv = 0;       // what the attention kernel sees (latent: kv_rank + rot_dim, kv_rank, 1)
    int           c_k = 0, c_v = 0, c_g = 0, c_rg1 = 0, c_rg2 = 0, c_router = 0;  // columns of the fused projection
    int           plain_stride = 0, lat_stride = 0;      // latent: head strides of the unrotated query parts / of the latent attention output
    DenseWeight   wo, gu, down;      // output projection; [gate | up] along N; down (experts: one image per expert in gu / down)
    DenseWeight   uk, uv;            // latent: key expansion transposed [kv_rank][dim] and value expansion [vdim][kv_rank], one image per head
    float *       r1 = nullptr, *r2 = nullptr, *rg1_b = nullptr, *rg2_b = nullptr, *c_norm = nullptr, *inv_freq = nullptr;
    // post-norm blocks (spec.post_norm): x += LN1(mixer(x)); x += LN2(ff(x)).  `qkv` holds every projection of the mixer's input side by
    // side (fp32 output), columns
    //   attention: [q | k | v]   lightning: [q | k | v | gate]   delta rule: [r | k | v | gate | removal rate | decay, inner part]
    bool               post = false;
    bool               shared_fused = false;    // the shared expert is one more item of the experts' batched products (shared_ff <= ff)
    int                c_end = 0;               // columns of the fused projection
    int                c_a = 0, c_w1 = 0;       // delta rule: columns of the removal-rate logits and of the decay's inner projection
    DenseWeight        w2, router, sh_up, sh_down;  // delta: decay outer projection; experts: router, shared expert
    float *            norm1_b = nullptr, *norm2_b = nullptr, *proj_bias = nullptr, *q_w = nullptr, *k_w = nullptr, *mix_norm = nullptr;
    float *            w0 = nullptr, *act_par = nullptr, *decay_d = nullptr;
    std::vector<float> decay_h;                 // lightning: the spec's decays (the spec's pointer is the caller's memory)
    size_t             state_offset = 0, state_floats = 0;  // this layer run's state inside a slot of the state pool (floats)
    // post-norm blocks with RMS group norms (spec.norm_groups): convolved projections, differential attention, and the parallel pair of a
    // biased attention (left) and a gated delta rule (right).  Fused projection columns
    //   attention: [q | k | v]                                 (two maps per query / key head with diff_maps)
    //   parallel:  [left q | left k | left gate | right q | right k | right v | beta | a1 (padded to 32) | g1]
    int          a_heads = 0;                  // query heads the attention kernel sees (two per head with diff_maps)
    int          a_kh = 0, a_vh = 0;           // key / value heads in the cache where they differ from a_kv (0: a_kv of each)
    bool         has_cache = true, has_state = false;
    int          conv_col = 0, conv_ch = 0, conv_taps = 0, conv_act = 0;  // the projection columns [conv_col, conv_col + conv_ch) pass a convolution
    float*       conv_w = nullptr;             // [conv_ch][taps]
    size_t       conv_offset = 0, conv_floats = 0;  // its state inside a slot of the state pool
    float *      lambda = nullptr, *dist_tab = nullptr, *talk = nullptr, *zero_sink = nullptr, *join_l = nullptr, *join_r = nullptr;
    int          dist_len = 0;
    int          c_rq = 0, c_rk = 0, c_rv = 0, c_b = 0, c_a1 = 0, c_g1 = 0;  // parallel: columns of the right mixer's projections
    int          c_xq = 0, c_xk = 0;           // ... and of its per-head query / key vectors behind the convolved columns
    int          r_nqk = 0, r_nv = 0, lora_g1 = 0;  // right: kv_heads * dim, heads * vdim; column of g1 among the cast inner activations
    DenseWeight  wo_r, a2, g2;
    float *      a_log = nullptr, *dt_bias = nullptr, *r_norm = nullptr;
};

struct LayeredModel {
    tm_layered_config    cfg{};
    std::vector<LmLayer> layers;
    DenseWeight          head;
    DenseWeight          loop_in;               // [width][2 width]: the mix of stream and embedding output at the start of a loop pass
    float*               loop_step = nullptr;   // [loop_times][width]
    void*                embed      = nullptr;  // [vocab][width] bf16 | fp32
    float*               final_norm = nullptr;
    int                  elem       = 2;        // bytes of an activation / cache element
    int                  ldw = 0, ldqkv = 0, ldcat = 0, ldv16 = 0;  // leading dimensions: normed rows, projections, [attention | ff], fp16 logits
    int                  ldproj = 0, ldq = 0, ldplain = 0, ldlat = 0, ldff = 0, ld2w = 0, max_top = 0;
    int                  max_logit_rows = 0;
    float*               d_res = nullptr;       // residual stream [max_tokens][width]
    void *               d_h1 = nullptr, *d_h2 = nullptr, *d_qkv = nullptr, *d_cat = nullptr, *d_hn = nullptr;
    // wide blocks: fused projection (fp32), queries, unrotated query parts, latent attention output, activations
    float *              d_proj = nullptr, *d_x0 = nullptr, *d_moe_y = nullptr, *d_topk_w = nullptr;
    void *               d_q = nullptr, *d_plain = nullptr, *d_lat = nullptr, *d_ff = nullptr, *d_xx = nullptr, *d_moe_x = nullptr;
    int *                d_topk_ids = nullptr, *d_offsets = nullptr, *d_f2n = nullptr, *d_en2f = nullptr;
    // post-norm blocks: a sublayer's fp32 result, state mixers' fp32 output and per-row vectors, the decay's inner activations
    float *              d_y = nullptr, *d_mixo = nullptr, *d_aux = nullptr, *d_wdec = nullptr, *final_norm_b = nullptr;
    float *              d_y2 = nullptr, *d_conv = nullptr, *d_gate2 = nullptr;  // the second branch's result, convolved projections, a gate
    int                  ldconv = 0;
    void*                d_lora = nullptr;
    int                  ldmix = 0, ldlora = 0;
    // recurrent states: [max_batch_size + 1 slots][state_slot_floats] fp32; the last slot takes the decode rows of slots without a sequence
    float*               d_state = nullptr;
    size_t               state_slot_floats = 0;
    bool                 has_post = false;
    float*               d_logits_f32 = nullptr;  // [max_logit_rows][vocab]
    int *                d_row_seq = nullptr, *d_row_pos = nullptr, *d_iota = nullptr, *d_want = nullptr, *d_seq_slot = nullptr;
    int *                d_step_ids = nullptr, *d_step_cu_q = nullptr, *d_step_k_len = nullptr;
    float*               d_attn_ws = nullptr;
    size_t               attn_ws_bytes = 0;
    int                  decode_splits = 1;
    int                  debug_layers  = -1;  // >= 0: the forward stops behind this many layers (parity tests read the residual stream)
    std::map<int64_t, int> sess_len;          // open sessions (scheduler request id) -> tokens held
    std::map<std::string, int> fan_in;        // tensor name -> input size (synthetic weights: N(0, 1 / fan_in))
};

// the rows of one forward that share a block table and a (cu_q, k_len) description
struct LmPart {
    int             row0, rows, nseq;
    const int*      cu_q;
    const int*      k_len;
    const int*      seq_slot;    // nullptr: sequence i -> table row i
    const uint64_t* block_ptrs;
    bool            decode;      // one row per sequence
    int             max_q_len;
    int             slot0  = 0;         // seq_slot == nullptr: sequence i lives in batch slot slot0 + i (the recurrent states are per slot)
    const int*      active = nullptr;   // [nseq] or nullptr; 0: a placeholder row of a slot without a running sequence
};

}  // namespace tmk

using namespace tmk;

struct tm_engine {
    tm_engine_config cfg{};
    // local (per-rank) dims
    int q_heads = 0, kv_heads = 0, inter = 0, vocab_local = 0, hidden = 0, D = 128;
    int qkv_n = 0;

    hipStream_t  stream = nullptr;
    ncclComm_t   comm   = nullptr;
    // TM_COMM_STREAM (default 1): the all-reduces of PREFILL-sized tensor-parallel forwards run on their own stream under the other
    // row half's GEMMs (engine_comm.hip: allreduce_rows_side; engine_forward.hip: forward_tail_two_halves).  Decode-sized forwards
    // keep every collective on the engine stream: a decode layer is one dependent chain, a side stream had nothing to run beside it
    // (profiles/r02_comm_stream_arms.txt; the fork / join arm of rounds 2-4 is gone)
    hipStream_t  comm_stream = nullptr;
    std::vector<hipEvent_t> pipe_events;      // (ready, done) pairs of the side-stream all-reduces of ONE forward
    size_t       pipe_events_used = 0;
    int          pipe_min_rows    = 1024;     // TM_PIPE_MIN_ROWS: smallest row half (forwards below twice this stay unsplit)
    int64_t      pipe_forwards = 0, pipe_mb_forwards = 0, pipe_allreduces = 0;   // tm_engine_comm_overlap_info
    // set by prefill_slots() around ONE forward: the forward's sequences [0, seqs_a) own its rows [0, rows_a) -- two micro-batches that
    // share nothing between the embedding and the lm_head (forward_layers_two_microbatches); seqs_a = 0: no such split (one sequence,
    // a lopsided boundary, a mixed forward) -> the row-half schedule inside every layer (forward_tail_two_halves)
    struct { int seqs_a = 0, rows_a = 0; } mb;
    float        emulate_ar_gbps = 0.f;       // TM_EMULATE_AR_GBPS, one-rank emulation only: stand-in for an exchange's duration (engine_comm.hip)
    // mixed forwards: the decode rows' attention runs on this stream beside the prefill rows' K/V store -> flatten -> attention
    // on the engine stream (reference: aux_stream_ + event fork / join, unified_attention_layer.cc:613-651)
    hipStream_t  aux_stream = nullptr;
    hipEvent_t   ev_aux_fork = nullptr, ev_aux_join = nullptr;
    bool         mixed_two_streams = true;  // TM_MIXED_2STREAM=0: back to back on the engine stream
    bool         mixed_steps_on    = true;  // TM_MIXED_STEP=0: prefill forwards and decode steps alternate
    bool         graph_comm        = true;  // TM_GRAPH_COMM=0: tensor-parallel decode steps stay eager (collectives not captured)
    // native communicator (TM_COMM=native, comm_p2p.hip): this rank's symmetric segment [flags 256 B | tile 0 | tile 1] and the
    // peers' mappings of theirs; serves the row-parallel all-reduces of forwards with M <= p2p_rows, RCCL the rest
    void*        p2p_seg = nullptr;
    void*        p2p_peer[8] = {};
    uint32_t*    p2p_state = nullptr;
    int          p2p_rows = 0;
    int          p2p_rows2 = 0;  // rows of the segment's two-shot regions (in2 / out2): forwards larger than p2p_rows (prefill) without RCCL
    bool         p2p_ready = false;
    bool         comm_overlap = false;   // TM_COMM_STREAM != 0 and an RCCL communicator: prefill all-reduces on comm_stream
    bool         graph_comm_failed = false;  // capturing the RCCL calls failed once: stay eager
    bool         use_comm = false;  // collectives on the data path: tp > 1 (or TM_FORCE_COMM=1: single-rank communicator,
                                    // exercises the RCCL code path on a 1-GPU box)
    std::map<std::string, Slot> slots;
    std::unique_ptr<tmk::LayeredModel> lm;   // set: a layer-list model (tm_engine_create_layered); `layers` below stays empty
    std::vector<Layer>          layers;
    half_t*      tok_embeddings = nullptr;
    half_t*      final_norm     = nullptr;
    LinearSlots  output;
    bool         weights_ready = false;
    bool         started       = false;

    // KV cache
    KvLayout  layout{};
    char*     pool        = nullptr;
    int64_t   block_bytes = 0;
    int64_t   num_blocks  = 0;
    std::vector<int> free_blocks;
    int       max_blocks_per_seq = 0;
    uint64_t* d_block_ptrs    = nullptr;  // [max_batch][max_blocks_per_seq]
    int*      d_cu_block_nums = nullptr;  // [max_batch+1]

    // activations
    int     max_tokens = 0;
    half_t *d_resid = nullptr, *d_x = nullptr, *d_qkv = nullptr, *d_attn = nullptr, *d_act = nullptr, *d_tmp = nullptr;
    half_t* d_logits = nullptr;
    half_t* d_last   = nullptr;
    float*  d_gemm_ws = nullptr;
    size_t  gemm_ws_bytes = 0;
    // RMSNorm folded into the decode GEMMs (NormFold, tm_kernels.h): per-tile sums of squares [hidden / 64][64] and the split-K
    // arrival counters of the producing GEMM; TM_FOLD_NORM=0 keeps the reduce-norm launches
    float*    d_ss      = nullptr;
    unsigned* d_tickets = nullptr;
    int       fold_max_rows = 64;  // rows of a forward up to which the folded layer runs (TM_FOLD_MAX_M: 64 | 128)
    int       fold_norm = 0;  // bit 0: wo -> w1w3, bit 1: w2 -> the next layer's w_qkv
    unsigned  h_mark = 0;             // host copy of the native communicator's give-up mark (device_marks_fetch)
    bool      comm_failed = false;    // a give-up mark was seen: the ranks' call sequences may have diverged (sticky, see device_marks_check)
    float*  d_attn_ws = nullptr;
    half_t *d_kflat = nullptr, *d_vflat = nullptr;
    int     kflat_stride = 0;
    half2_t* d_rope = nullptr;
    int      rope_max_pos = 0;

    // batch state (device)
    int *d_next_ids = nullptr;
    int *d_ids = nullptr, *d_k_len = nullptr, *d_cu_q = nullptr, *d_cu_koff = nullptr, *d_rows = nullptr;
    int *d_cu_q_b = nullptr;   // cu_q of the second micro-batch of a tensor-parallel prefill forward, counted from ITS first row
    int *d_generated = nullptr, *d_step = nullptr;
    int *d_prefill_ids = nullptr;
    half_t* d_argmax_val = nullptr;
    float*  d_cand = nullptr;
    float*  d_cand_all = nullptr;

    // batch state (host)
    int              batch = 0, max_new = 0;
    std::vector<int> h_len;
    std::vector<std::vector<int>> h_blocks;
    int              steps_done = 0;
    int              steps_fetched = 0;  // steps_done at the last fetch that saw no communicator give-up mark
    int              steps_valid = -1;   // >= 0 after a give-up: the columns of d_generated known to be valid

    int            decode_splits = 1;
    bool           fuse_qkv      = false;  // decode: qkv GEMM output -> attention kernel directly (int8 KV, MFMA kernel)
    hipGraphExec_t graph = nullptr;
    // per-kernel-category HIP event profiling (tm_engine_profile_decode)
    bool                                            prof_on = false;
    std::vector<hipEvent_t>                         prof_pool;
    size_t                                          prof_used = 0;
    std::vector<std::tuple<int, size_t, size_t>>    prof_spans;  // (category, start event, stop event)
    std::vector<float>                              h_ttft_ms;
    int            graph_batch = 0;
    int            graph_max_new = 0;  // record_kernel's bound is a captured kernel argument

    // continuous batching (tm_engine_submit / step / poll / cancel): slot-based, every decode step runs all
    // max_batch_size slots; free slots are parked on a scratch block with k_len = 1 and never advance
    std::unique_ptr<tmk::BatchScheduler> sched;
    int64_t          mixed_steps = 0;        // scheduler steps whose decode rows rode on a prefill forward
    int*             d_active    = nullptr;  // [max_batch] 1 = slot holds a running sequence
    uint64_t*        d_pf_block_ptrs = nullptr;  // [max_batch][max_blocks_per_seq] the table an admission's prefill walks: a new
                                                 // slot's row reaches the decode table (d_block_ptrs) only once it is prefilled,
                                                 // until then its decode row stays parked on the dummy block (a mixed forward runs
                                                 // the parked decode row and the real prefill of the same slot side by side)
    int*             d_pf_k_len  = nullptr;  // prefill-local arrays (the decode arrays stay live during an admission)
    int*             d_pf_cu_q   = nullptr;
    int*             d_first_ids = nullptr;  // [max_batch] first tokens of an admission's earlier prefill iterations (mixed steps)
    std::vector<int> h_active;
    int              dummy_block = -1;
    hipGraphExec_t   graph_cb    = nullptr;
    // Two-phase schedule / forward overlap (reference: the two alternating batch phases of turbomind.cc:171, engine.cc:770-870):
    // a pure decode step is ISSUED (graph launch + result copy into a pinned buffer + event) and RETIRED (event wait, tokens to
    // the scheduler, finished slots parked) by different scheduler steps -- step N+1 is issued before step N is retired, so the
    // host's bookkeeping, the caller's polling and the next launch run under the device's step N+1.  A sequence that ends in
    // step N rides one more step as a dead row (its token is dropped: the slot's request id no longer matches).
    // TM_ASYNC_STEP=1 switches the overlap on; by default every step is retired by the call that issued it (see cb_enter).
    struct PendingStep {
        bool                 valid = false;
        bool                 lp    = false;  // the step's logprob records were copied into the pinned buffers of `buf` as well
        int                  buf   = 0;
        std::vector<int64_t> ids;  // request of every slot whose token this step produces (-1: free, parked, prefilled by this step)
    } pending;
    bool       async_step_on = false;
    int*       h_step_pin[2] = {nullptr, nullptr};  // pinned [max_batch + 1]: next ids of the slots, then the communicator's give-up mark
    hipEvent_t ev_step[2]    = {nullptr, nullptr};
    int        issue_count   = 0;
    int64_t    overlapped_steps = 0;  // decode steps issued while the previous one was still unretired

    // stochastic sampling (tm_engine_set_sampling / tm_engine_submit_ex); off = arg-max
    bool      sampling_on = false, graph_sampling = false, graph_cb_sampling = false;
    float *   d_temp = nullptr, *d_topp = nullptr, *d_minp = nullptr, *d_u = nullptr;
    int*      d_topk = nullptr;
    uint64_t* d_seed = nullptr;
    void*     d_sample_ws = nullptr;
    half_t*   d_logits_gather = nullptr;  // tp > 1 + sampling: [tp][max_batch][vocab / tp] all-gathered shards ...
    half_t*   d_logits_full   = nullptr;  // ... and the full rows [max_batch][vocab] every rank samples from
    void*     d_moe_ws    = nullptr;  // routing tables + expert activations of one forward (moe_workspace_bytes)
    // logprobs of the generated tokens (tm_engine_set_logprobs, static batch): records [batch][max_new] x [cap] next to d_generated
    int    logprobs_next = 0, logprobs_n = 0;
    bool   logprobs_on = false, graph_logprobs = false;
    float *d_lpr_vals = nullptr, *d_lpr_sel = nullptr;
    int *  d_lpr_idx = nullptr, *d_lpr_num = nullptr, *d_kept = nullptr;
    size_t lpr_records = 0, lpr_entries = 0;  // allocated records / records x cap
    // continuous batching (tm_engine_request_logprobs): the record of the CURRENT step per batch slot, [max_batch][kMaxLogProb] on the
    // device, copied behind every step into the pinned buffer of the step's parity (first cb_lp_used columns) and appended to the
    // requests that asked for logprobs when the step is retired
    bool   cb_logprobs_on = false, graph_cb_logprobs = false;
    int    cb_lp_used = 0;
    float *d_cb_lp_vals = nullptr, *d_cb_lp_sel = nullptr, *h_cb_lp_vals[2] = {nullptr, nullptr}, *h_cb_lp_sel[2] = {nullptr, nullptr};
    int *  d_cb_lp_idx = nullptr, *d_cb_lp_num = nullptr, *h_cb_lp_idx[2] = {nullptr, nullptr}, *h_cb_lp_num[2] = {nullptr, nullptr};
    std::vector<tm_sampling>       h_sampling;      // static batch: parameters of the next prefill
    std::map<int64_t, tm_sampling> cb_sampling;     // continuous batching: per request

    // logits processors (tm_engine_set_logits_params / tm_engine_submit_gen): repetition penalty, bad ids, min length;
    // off = arg-max / sampling see the raw lm_head output.  d_seen = persistent "token occurs in the sequence" bitmask
    // per batch slot over the GLOBAL vocabulary.
    bool      logits_on = false, graph_logits = false, graph_cb_logits = false;
    uint32_t* d_seen     = nullptr;
    int       seen_words = 0;
    float*    d_lp_rep    = nullptr;
    int *     d_lp_minlen = nullptr, *d_lp_ban = nullptr, *d_lp_end = nullptr;
    std::vector<tm_logits_param>       h_logits;   // static batch: parameters of the next prefill
    std::map<int64_t, tm_logits_param> cb_logits;  // continuous batching: per request

    // engine thread (tm_engine_serve_start): runs step_locked() while requests exist.  `mu` serialises the scheduler
    // and every device-side effect of submit / step / poll / cancel; API callers announce themselves in api_waiting so
    // that the loop (which re-locks immediately) lets them in between two steps.
    std::mutex              mu;
    std::condition_variable cv_work, cv_out;
    std::thread             loop;
    std::atomic<int>        api_waiting{0};
    std::atomic<bool>       loop_on{false};
    bool                    loop_stop = false;
    int                     loop_rc   = 0;
    std::string             loop_err;
    tm_request_cb           on_update      = nullptr;
    void*                   on_update_user = nullptr;
};

namespace tmk {

// lock of an API call: counted, so that the engine thread yields to callers between steps
struct ApiLock {
    tm_engine*                   e;
    std::unique_lock<std::mutex> lk;
    explicit ApiLock(tm_engine* eng): e(eng), lk(eng->mu, std::defer_lock)
    {
        e->api_waiting.fetch_add(1);
        lk.lock();
        e->api_waiting.fetch_sub(1);
    }
};

struct StepUpdate {
    int64_t id;
    int     status, n_tokens;
};

enum ProfCat { P_EMBED = 0, P_GEMM_QKV, P_KV_STORE, P_ATTN, P_GEMM_O, P_RES_NORM, P_GEMM_GATE_UP, P_GEMM_DOWN, P_LM_HEAD,
               P_SAMPLE, P_ALLREDUCE, P_NUM };

#define TM_PROF(cat, stmt)                                                                         \
    do {                                                                                           \
        size_t _a = 0;                                                                             \
        if (e->prof_on) {                                                                          \
            _a = prof_event(e);                                                                    \
        }                                                                                          \
        stmt;                                                                                      \
        if (e->prof_on) {                                                                          \
            e->prof_spans.emplace_back((int)(cat), _a, prof_event(e));                             \
        }                                                                                          \
    } while (0)

// the decode rows of a mixed forward (forward(), engine_forward.hip)
struct MixedDecode {
    int             rows;        // decode rows = batch slots
    const int*      k_len;       // [rows] context lengths including this step's token
    const uint64_t* block_ptrs;  // the unshifted block table
    const int*      cu_q;        // [rows + 1] = 0 .. rows (one token per decode row; kv_rope_store of the fp16-KV path)
    const int*      active;      // [rows] 1 = the slot holds a running sequence (logits processors skip the others)
};

// the decode step that rides on the last prefill forward of a continuous-batching admission (prefill_slots(), engine_forward.hip)
struct MixedStep {
    int        rows;     // batch slots = decode rows
    int*       k_len;    // the decode state arrays (NOT the iteration-local e->d_k_len)
    const int* active;
    int*       ids;      // current token of every slot
    const uint64_t* block_ptrs;  // the decode block table
    const int* cu_q;     // 0 .. rows (the decode step's own array)
    bool*      done;
};

template<class T>
inline int dmalloc(T** p, size_t n)
{
    TM_HIP_CHECK(hipMalloc((void**)p, n * sizeof(T)));
    return 0;
}

// ---- shared between the engine translation units ----
int launch_advance_active(int* k_len, const int* active, int n, hipStream_t st);
size_t prof_event(tm_engine* e);
void p2p_tables(tm_engine* e, half_t** data, uint32_t** flags);
int reduce_residual_norm(tm_engine* e, int M, const half_t* norm_w);
bool prefill_pipe_ok(const tm_engine* e, int M);
int allreduce_rows_side(tm_engine* e, int r0, int rows, hipEvent_t* done);
int pipe_wait(tm_engine* e, hipEvent_t done);
int forward(tm_engine* e, const int* d_ids, int M, int nseq, bool decode, int max_q_len, int max_k_len, int kflat_stride, int slot0,
            const MixedDecode* md = nullptr);
int sample_rows(tm_engine* e, int n, int slot, const int* ids_in, const int* cu_q, int ntok, const int* k_len, const int* active);
int layered_forward(tm_engine* e, const int* d_ids, int M, int nseq, bool decode, int max_q_len, int max_k_len, int slot0, const MixedDecode* md);
int layered_process_weights(tm_engine* e);
int layered_init_synthetic(tm_engine* e, uint64_t seed);
int layered_start(tm_engine* e);
void layered_free(tm_engine* e);
int device_marks_fetch(tm_engine* e, bool async);
int device_marks_check(tm_engine* e);

}  // namespace tmk

extern "C" {

extern const tm_logits_param kNoLogitsParam;  // every logits processor off (engine_forward.hip)

int tune_decode_gemms(tm_engine* e, int M, bool verbose);
int sampling_upload(tm_engine* e, const tm_sampling* p, int slot0, int n);
int logits_param_check(const tm_logits_param& p);
int logits_upload(tm_engine* e, const tm_logits_param* p, const int* prompt_len, const int* eos, int slot0, int n);
void setup_decode(tm_engine* e, int batch);
int prefill_slots(tm_engine* e, const int* const* seq_ids, const int* host_lens, int batch, int slot0, float* ttft_ms,
                  const MixedStep* mix = nullptr);
bool graph_enabled(const tm_engine* e);
int cb_enter(tm_engine* e);  // switch the engine into continuous-batching mode (scheduler, parked slots); idempotent
int capture_step(tm_engine* e, int (*step)(tm_engine*), hipGraphExec_t* exec);

}  // extern "C"
