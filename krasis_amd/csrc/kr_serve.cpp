// kr_serve.cpp -- the batched serving store behind kr_serve_* (include/krasis_hip.h): weights in bf16 or f32, a page pool shared by the request
// slots, and the step function that runs a ragged batch (prompt portions beside single decoded tokens) through every layer.
//
// Memory: one K and one V pool per layer that owns a cache, [pages][page_tokens][kv_heads * dim | vdim]; a layer that borrows another layer's
// keys / values points at that layer's pools.  A slot holds the list of its pages; the device copy of the table ([max_slots][pages]) is refreshed
// at the start of a step.  Scratch buffers grow to the largest step seen and are then reused (no allocation in a steady state).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include "kr_engine_internal.h"
#include "kr_sampler.h"
#include "kr_serve_ops.h"

namespace {
struct SvLayer {
    kr_serve_layer d{};
    // hw: every matrix that multiplies the normed input, row blocks [q | k | v | router | gate | up] (router: E rows, or hi + lo = 2E rows in a bf16
    // store; gate | up: the dense feed-forward's or the shared expert's) -- one GEMM per layer produces them all
    // A latent mixer's first row blocks are [dq | dkv] instead of [q | k | v]; its up-projections are matrices of their own: uq, and per head ukT
    // [kv_rank, dim] (W_uk of the head transposed: it multiplies the QUERY) and uv [vdim, kv_rank].
    DevBuf norm_w, norm_b, norm2_w, norm2_b, post1_w, post1_b, post2_w, post2_b, hw, o, sink, down, egu, edown, sdown, kpool, vpool;
    DevBuf q_norm, k_norm, vmix, router_b, slopes, dq_norm, dkv_norm, uq, ukT, uv;
    // biases of q / k / o; the input convolution's taps and its per-slot rows; the residual gates (the mixer's is a matrix of its own: it multiplies the
    // un-convolved input; the feed-forward's is the last row block of hw); recurrent mixers: output norm weight, decays, gate biases, per-slot state
    DevBuf q_bias, k_bias, o_bias, canon, canon_state, rg1, rg1_b, rg2_b, lin_norm, decay, i_bias, f_bias, lin_state, lin_nm;
    size_t lin_state_stride = 0, lin_nm_stride = 0;
    // the vector that joins the stream before the layer; the value bias; the short convolution on q | k | v: taps [nq + nk + nv, taps], the projections'
    // biases as one vector for it, its per-slot ring; the decay projections of a gla mixer (a1 feeds a2 in the storage type, so it is a matrix of its own)
    DevBuf pre_add, v_bias, pconv_w, pconv_bias, pconv_state, a1, a2, a2_b;
    // state-space mixer: convolution taps and bias, dt bias, log rates, skip weights, norm weight; per slot the convolution's ring and S [heads][vdim][state]
    DevBuf sconv_w, sconv_b, dt_bias, a_log, ssd_d, ssd_norm, sconv_state, ssd_state;
    size_t ssd_state_stride = 0;
    int wsrc = 0;                // the layer whose tensors this one uses (itself, or d.weights_of - 1); cache pools and state are always the layer's own
    // row blocks of hw: mixer [q | k | v | out gate | i | f | state-space in-projection] (n_qkv rows in all), then [router | gate | up | residual gate of the feed-forward]
    int rope_id = 0, n_qkv = 0, off_ogate = 0, off_if = 0, off_ssd = 0, off_router = 0, n_router = 0, off_gu = 0, n_gu = 0, off_rg2 = 0, n_h = 0;
    bool latent() const { return d.mixer_kind == KR_SERVE_MIX_LATENT; }
    bool gla() const { return d.mixer_kind == KR_SERVE_MIX_GLA; }
    bool recurrent() const { return d.mixer_kind == KR_SERVE_MIX_RETENTION || d.mixer_kind == KR_SERVE_MIX_MLSTM || gla(); }
    bool chunkable() const { return d.mixer_kind == KR_SERVE_MIX_RETENTION || d.mixer_kind == KR_SERVE_MIX_MLSTM; }      // the block form of the recurrence
    bool ssd_alone() const { return d.mixer_kind == KR_SERVE_MIX_SSD; }
    bool has_ssd() const { return ssd_alone() || d.side_mixer == KR_SERVE_MIX_SSD; }
    int ssd_inner() const { return d.ssd_heads * d.ssd_vdim; }
    int ssd_conv_c() const { return ssd_inner() + 2 * d.ssd_groups * d.ssd_state; }
    int ssd_in_rows() const { return 2 * ssd_inner() + 2 * d.ssd_groups * d.ssd_state + d.ssd_heads; }
    int att_out_cols() const { return ssd_alone() ? 0 : d.heads * d.vdim; }                   // the output projection reads [first mixer | state-space mixer]
    int o_cols() const { return att_out_cols() + (has_ssd() ? ssd_inner() : 0); }
    int pconv_c() const { return d.heads * d.dim + d.kv_heads * (d.dim + d.vdim); }
    bool ungated_ff() const { return d.dense_act == KR_SERVE_ACT_RELU2; }
    bool has_cache() const { return !recurrent() && !ssd_alone() && d.kv_from < 0; }
    int att_heads_kv() const { return latent() ? 1 : d.kv_heads; }
    int att_dim() const { return latent() ? d.kv_rank + d.rot_dims : d.dim; }       // key row of the attention kernels
    int att_vdim() const { return latent() ? d.kv_rank : d.vdim; }
    std::vector<char> have;      // per role (expert roles: one flag per expert)
    int have_eg = 0, have_eu = 0, have_ed = 0;
    std::vector<char> eg, eu, ed;
};
struct SvRope { int dims, scaling; double base, factor, original, fast, slow; float mult; DevBuf inv_freq; DevBuf cs; };
struct SvSlot { bool live = false; int len = 0; int last_token = -1; std::vector<int> pages; };      // last_token: the pair embedding's previous token
}  // namespace

struct kr_serve {
    int device = 0;
    kr_serve_config c{};
    bool f32 = false, finalized = false;
    size_t esz = 2;
    hipStream_t st = nullptr;
    std::vector<SvLayer> L;
    std::vector<SvRope> ropes;
    DevBuf embed, head, fnorm_w, fnorm_b, enorm_w, bigram;
    bool have_embed = false, have_head = false, have_fw = false, have_fb = false, have_enorm = false, have_bigram = false;
    // cache
    int n_pages = 0;
    std::vector<int> free_pages;
    std::vector<SvSlot> slots;
    DevBuf page_table;
    std::vector<int> h_table;
    // step scratch
    DevBuf meta, x, h, qkv, att, mix, gu, y, rows, ffout, ids, wts, rz, moe_i, hw, logits, amax, part_ml, part_acc;
    // f32 copy of the mixer's normed input, its convolved form, residual gate logits, whole-row q / k statistics, recurrent outputs; chunked recurrence:
    // per-token gate terms, state / normaliser at every block's start, per-block gate terms
    DevBuf h32, hc, rg, qk_rms, lin_o, lin_tok, lin_sbuf, lin_nbuf, lin_cm;
    DevBuf ssd_z;                                         // the state-space mixer's rows in the block recurrence's layout [q | k | v] per head (prompt portions)
    DevBuf qkv2, sconv, ga1, gz;                          // convolved q | k | v; convolved x | B | C; the gla decay's low-rank input (storage type) and logits
    DevBuf v_first;                                      // [T, kv_heads * vdim] f32: the values of the first value-mixing layer
    DevBuf lq_c, lq_2, lq_n, lq_e, att2, head_i;         // latent mixer: query latent, W_uq output, plain query parts, folded queries, per-head values, head row tables
    void* h_meta = nullptr; size_t h_meta_bytes = 0;     // pinned staging of the per-step arrays
    int last_want = 0;
    // capture / profile
    bool capture = false; DevBuf cap; int cap_T = 0;
    bool prof = false; double prof_ms[8] = {0}; hipEvent_t ev0 = nullptr, ev1 = nullptr;
    // decode-shaped steps repeat with the same launch sequence: captured once into a hipGraph, replayed afterwards
    struct Graph { uint64_t key; hipGraphExec_t exec; };
    std::vector<Graph> graphs;
    std::vector<std::pair<uint64_t, int>> seen;      // keys met so far (a shape is captured at its second visit)
    bool use_graph = true; long graph_replays = 0;
    // sampler scratch
    DevBuf s_keys, s_sorted, s_temp, s_probs, s_rng, s_tok, s_seen, s_row;
    size_t weight_bytes = 0;
};

namespace {
uint16_t f32_to_bf16_host(float f) {
    uint32_t b; std::memcpy(&b, &f, 4);
    if ((b & 0x7F800000u) == 0x7F800000u && (b & 0x7FFFFFu)) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7FFFu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}
float bf16_to_f32_host(uint16_t v) { uint32_t b = (uint32_t)v << 16; float f; std::memcpy(&f, &b, 4); return f; }

// host [n] of src_dtype -> device at dst + offset elements, as f32 (to_f32) or in the store's type
int upload(kr_serve* s, DevBuf& dst, size_t total_elems, size_t offset_elems, const void* host, int src_dtype, size_t n, bool to_f32) {
    const size_t esz = to_f32 ? 4 : s->esz;
    if (!dst.p) {
        if (dst.ensure(total_elems * esz)) return kr_fail(KR_ERR_HIP, "hipMalloc of %zu bytes failed", total_elems * esz);
        s->weight_bytes += total_elems * esz;
    }
    if ((offset_elems + n) * esz > dst.bytes) return kr_fail(KR_ERR_VALUE, "tensor does not fit its slot");
    const bool want_f32 = to_f32 || s->f32;
    std::vector<char> tmp;
    const void* src = host;
    if (want_f32 && src_dtype == KR_SERVE_BF16) {
        tmp.resize(n * 4); float* o = (float*)tmp.data(); const uint16_t* i = (const uint16_t*)host;
        for (size_t k = 0; k < n; k++) o[k] = bf16_to_f32_host(i[k]);
        src = tmp.data();
    } else if (!want_f32 && src_dtype == KR_SERVE_F32) {
        tmp.resize(n * 2); uint16_t* o = (uint16_t*)tmp.data(); const float* i = (const float*)host;
        for (size_t k = 0; k < n; k++) o[k] = f32_to_bf16_host(i[k]);
        src = tmp.data();
    }
    KR_HIP(hipMemcpy((char*)dst.p + offset_elems * esz, src, n * esz, hipMemcpyHostToDevice));
    return KR_OK;
}

// host [rows, cols] -> columns [col0, col0 + cols) of the device matrix dst [rows, total_cols] in the store's type
int upload_cols(kr_serve* s, DevBuf& dst, size_t rows, size_t total_cols, size_t col0, const void* host, int src_dtype, size_t cols) {
    const size_t esz = s->esz, n = rows * cols;
    if (!dst.p) {
        if (dst.ensure(rows * total_cols * esz)) return kr_fail(KR_ERR_HIP, "hipMalloc of %zu bytes failed", rows * total_cols * esz);
        s->weight_bytes += rows * total_cols * esz;
    }
    if (col0 + cols > total_cols || rows * total_cols * esz > dst.bytes) return kr_fail(KR_ERR_VALUE, "tensor does not fit its slot");
    std::vector<char> tmp;
    const void* src = host;
    if (s->f32 && src_dtype == KR_SERVE_BF16) {
        tmp.resize(n * 4); float* o = (float*)tmp.data(); const uint16_t* i = (const uint16_t*)host;
        for (size_t k = 0; k < n; k++) o[k] = bf16_to_f32_host(i[k]);
        src = tmp.data();
    } else if (!s->f32 && src_dtype == KR_SERVE_F32) {
        tmp.resize(n * 2); uint16_t* o = (uint16_t*)tmp.data(); const float* i = (const float*)host;
        for (size_t k = 0; k < n; k++) o[k] = f32_to_bf16_host(i[k]);
        src = tmp.data();
    }
    KR_HIP(hipMemcpy2D((char*)dst.p + col0 * esz, total_cols * esz, src, cols * esz, cols * esz, rows, hipMemcpyHostToDevice));
    return KR_OK;
}
// a norm weight [n] as f32 with the design's offset added (weights stored around zero: offset 1)
int upload_norm_w(kr_serve* s, DevBuf& dst, const void* host, int src_dtype, size_t n) {
    std::vector<float> w(n);
    for (size_t k = 0; k < n; k++) w[k] = (src_dtype == KR_SERVE_F32 ? ((const float*)host)[k] : bf16_to_f32_host(((const uint16_t*)host)[k])) + s->c.norm_weight_offset;
    return upload(s, dst, n, 0, w.data(), KR_SERVE_F32, n, true);
}

int check_layer(const kr_serve_config& c, const kr_serve_layer* all, int i) {
    const kr_serve_layer& d = all[i];
    const bool ssd1 = d.mixer_kind == KR_SERVE_MIX_SSD, ssd = ssd1 || d.side_mixer == KR_SERVE_MIX_SSD;
    if (d.side_mixer != 0 && d.side_mixer != KR_SERVE_MIX_SSD) return kr_fail(KR_ERR_VALUE, "layer %d: side mixer %d", i, d.side_mixer);
    if (d.side_mixer && d.mixer_kind != KR_SERVE_MIX_ATTENTION) return kr_fail(KR_ERR_VALUE, "layer %d: a side mixer stands beside an attention mixer", i);
    if (ssd) {
        if (d.ssd_heads < 1 || d.ssd_vdim < 1 || d.ssd_vdim > 512 || d.ssd_state < 1 || d.ssd_state > 512 || d.ssd_groups < 1 || d.ssd_heads % d.ssd_groups || d.ssd_conv < 1 || d.ssd_conv > 64 ||
            d.ssd_norm_groups < 1 || (d.ssd_heads * d.ssd_vdim) % d.ssd_norm_groups)
            return kr_fail(KR_ERR_VALUE, "layer %d: state-space sizes (heads %d, vdim %d, state %d, groups %d, taps %d, norm groups %d)", i, d.ssd_heads, d.ssd_vdim, d.ssd_state, d.ssd_groups,
                           d.ssd_conv, d.ssd_norm_groups);
    }
    if (d.weights_of < 0 || d.weights_of > i) return kr_fail(KR_ERR_VALUE, "layer %d: weights_of %d is not an earlier layer", i, d.weights_of);
    if (d.weights_of) {
        kr_serve_layer a = d, b = all[d.weights_of - 1];
        if (b.weights_of) return kr_fail(KR_ERR_VALUE, "layer %d: layer %d does not own its tensors", i, d.weights_of - 1);
        a.weights_of = b.weights_of = 0; a.pre_add = b.pre_add = 0;
        if (std::memcmp(&a, &b, sizeof a) != 0) return kr_fail(KR_ERR_VALUE, "layer %d: its description differs from layer %d whose tensors it uses", i, d.weights_of - 1);
        if (d.kv_from >= 0 || d.v_mix) return kr_fail(KR_ERR_VALUE, "layer %d: a layer that runs again keeps a cache of its own and mixes no values", i);
    }
    if (d.pre_add && (!c.pre_norm || c.canon_taps > 1)) return kr_fail(KR_ERR_VALUE, "layer %d: a vector before the layer needs pre-normed blocks without an input convolution", i);
    if (d.dense_act < 0 || d.dense_act > KR_SERVE_ACT_RELU2 || d.expert_act == KR_SERVE_ACT_RELU2) return kr_fail(KR_ERR_VALUE, "layer %d: activation %d / %d", i, d.dense_act, d.expert_act);
    if (d.dense_act == KR_SERVE_ACT_RELU2 && c.res_gate) return kr_fail(KR_ERR_VALUE, "layer %d: the un-gated feed-forward has no gated residual", i);
    if (ssd1) {
        if (d.kv_from >= 0 || d.v_mix || d.qk_unit_norm || d.window || d.chunk || d.has_sink || d.dist_bias || d.proj_bias || d.v_from_k || d.out_gate || d.softcap != 0.0f || d.rot_dims ||
            d.proj_conv || d.gate_cap != 0.0f || d.lin_norm_weight)
            return kr_fail(KR_ERR_VALUE, "layer %d: an attention-only mechanism is switched on for a state-space mixer", i);
    } else {
    if (d.heads < 1 || d.kv_heads < 1 || d.heads % d.kv_heads) return kr_fail(KR_ERR_VALUE, "layer %d: heads %d / kv_heads %d", i, d.heads, d.kv_heads);
    if (d.dim < 1 || d.vdim < 1 || d.vdim > 512 || d.dim > 512) return kr_fail(KR_ERR_VALUE, "layer %d: head sizes %d / %d (at most 512)", i, d.dim, d.vdim);
    const bool lat = d.mixer_kind == KR_SERVE_MIX_LATENT;
    const bool rec = d.mixer_kind == KR_SERVE_MIX_RETENTION || d.mixer_kind == KR_SERVE_MIX_MLSTM || d.mixer_kind == KR_SERVE_MIX_GLA;
    if (d.mixer_kind != KR_SERVE_MIX_ATTENTION && !lat && !rec) return kr_fail(KR_ERR_VALUE, "layer %d: mixer kind %d", i, d.mixer_kind);
    if (d.mixer_kind == KR_SERVE_MIX_GLA && (d.decay_rank < 1 || !(d.decay_tau > 0.0f) || d.lin_norm_weight != 2)) return kr_fail(KR_ERR_VALUE, "layer %d: gla needs decay_rank, decay_tau and a shared norm weight", i);
    if (d.mixer_kind != KR_SERVE_MIX_GLA && (d.decay_rank || d.decay_tau != 0.0f)) return kr_fail(KR_ERR_VALUE, "layer %d: decay_rank / decay_tau belong to the gla mixer", i);
    if (d.proj_conv < 0 || d.proj_conv > 64 || (d.proj_conv && (d.mixer_kind != KR_SERVE_MIX_ATTENTION || d.kv_from >= 0 || d.v_from_k || d.v_mix || d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE)))
        return kr_fail(KR_ERR_VALUE, "layer %d: the convolution on q / k / v needs an attention mixer with projections and a cache of its own, per-head norms, no value mixing", i);
    if (d.proj_bias < 0 || d.proj_bias > 2 || (d.proj_bias == 2 && (d.v_from_k || d.kv_from >= 0))) return kr_fail(KR_ERR_VALUE, "layer %d: projection biases %d", i, d.proj_bias);
    if (rec) {
        if (d.kv_heads != d.heads) return kr_fail(KR_ERR_VALUE, "layer %d: a recurrent mixer has one key / value head per query head", i);
        if (d.kv_from >= 0 || d.v_mix || d.qk_unit_norm || d.window || d.chunk || d.has_sink || d.dist_bias || d.proj_bias || d.v_from_k || d.out_gate || d.softcap != 0.0f)
            return kr_fail(KR_ERR_VALUE, "layer %d: an attention-only mechanism is switched on for a recurrent mixer", i);
        if (d.rot_dims && (d.rot_interleaved || d.mixer_kind != KR_SERVE_MIX_RETENTION)) return kr_fail(KR_ERR_VALUE, "layer %d: recurrent mixers rotate half-split pairs, retention only", i);
    } else if (d.gate_cap != 0.0f || d.lin_norm_weight) return kr_fail(KR_ERR_VALUE, "layer %d: gate_cap / lin_norm_weight belong to recurrent mixers", i);
    if (d.v_from_k && (lat || d.vdim != d.dim || d.v_mix || d.kv_from >= 0)) return kr_fail(KR_ERR_VALUE, "layer %d: values that are the keys need vdim == dim, a cache of their own and no value mixing", i);
    if ((d.proj_bias || d.out_gate) && lat) return kr_fail(KR_ERR_VALUE, "layer %d: a latent mixer has no projection biases / output gate", i);
    if (d.out_gate < 0 || d.out_gate > KR_SERVE_OGATE_ELEM_SIGMOID || d.softcap < 0.0f || d.router_bias < 0 || d.router_bias > KR_SERVE_RBIAS_CHOICE || d.router_score < 0 ||
        d.router_score > KR_SERVE_RSCORE_SIGMOID || d.group_score < 0 || d.group_score > KR_SERVE_GSCORE_TOP2)
        return kr_fail(KR_ERR_VALUE, "layer %d: output gate %d / softcap %g / router bias %d / score %d / group score %d", i, d.out_gate, (double)d.softcap, d.router_bias, d.router_score, d.group_score);
    if (d.rot_dims < 0 || (!lat && d.rot_dims > d.dim) || (d.rot_dims & 1)) return kr_fail(KR_ERR_VALUE, "layer %d: rot_dims %d of %d", i, d.rot_dims, d.dim);
    if (d.rot_dims && (!(d.rot_base > 0.0) || !(d.rot_factor > 0.0))) return kr_fail(KR_ERR_VALUE, "layer %d: rotation base / factor", i);
    if (d.rot_scaling != KR_SERVE_ROT_LINEAR && d.rot_scaling != KR_SERVE_ROT_BY_PARTS && d.rot_scaling != KR_SERVE_ROT_BANDS) return kr_fail(KR_ERR_VALUE, "layer %d: rotation scaling %d", i, d.rot_scaling);
    if (d.rot_dims && d.rot_scaling == KR_SERVE_ROT_BANDS && (!(d.rot_original > 0.0) || !(d.rot_slow > 0.0) || !(d.rot_fast > d.rot_slow)))
        return kr_fail(KR_ERR_VALUE, "layer %d: banded rotation scaling needs original > 0 and fast > slow > 0", i);
    if (d.rot_dims && d.rot_scaling == KR_SERVE_ROT_BY_PARTS && (!(d.rot_original > 0.0) || !(d.rot_fast > 0.0) || !(d.rot_slow > 0.0) || !(d.rot_base > 1.0)))
        return kr_fail(KR_ERR_VALUE, "layer %d: by-parts rotation scaling needs original, fast, slow > 0 and base > 1", i);
    if (d.window < 0 || d.chunk < 0 || (d.window > 0 && d.chunk > 0)) return kr_fail(KR_ERR_VALUE, "layer %d: window %d / chunk %d", i, d.window, d.chunk);
    if (d.qk_unit_norm < 0 || d.qk_unit_norm > KR_SERVE_QKNORM_WHOLE || d.has_sink < 0 || d.has_sink > KR_SERVE_SINK_ZERO || d.v_mix < 0 || d.v_mix > KR_SERVE_VMIX_BLEND)
        return kr_fail(KR_ERR_VALUE, "layer %d: qk norm %d / sink %d / value mixing %d", i, d.qk_unit_norm, d.has_sink, d.v_mix);
    if (lat) {
        if (d.q_rank < 1 || d.kv_rank < 1 || d.kv_rank > 512 || d.kv_rank + d.rot_dims > 1024) return kr_fail(KR_ERR_VALUE, "layer %d: latent sizes %d / %d", i, d.q_rank, d.kv_rank);
        if (d.kv_from >= 0 || d.v_mix || d.qk_unit_norm || d.kv_heads != 1) return kr_fail(KR_ERR_VALUE, "layer %d: a latent mixer has one latent per token, no borrowed cache, no value mixing, no q / k norm", i);
    }
    if (d.v_mix == KR_SERVE_VMIX_BLEND) {
        int src = -1;
        for (int j = 0; j < i; j++) if (all[j].v_mix == KR_SERVE_VMIX_FIRST) { src = j; break; }
        if (src < 0) return kr_fail(KR_ERR_VALUE, "layer %d mixes values but no earlier layer keeps its own", i);
        if (all[src].kv_heads * all[src].vdim != d.kv_heads * d.vdim) return kr_fail(KR_ERR_VALUE, "layer %d: values of layer %d have another size", i, src);
    }
    if (d.v_mix && d.kv_from >= 0) return kr_fail(KR_ERR_VALUE, "layer %d: value mixing needs values of its own", i);
    if (d.kv_from >= 0) {
        if (d.kv_from >= i) return kr_fail(KR_ERR_VALUE, "layer %d: kv_from %d is not an earlier layer", i, d.kv_from);
        const kr_serve_layer& o = all[d.kv_from];
        if (o.kv_from >= 0) return kr_fail(KR_ERR_VALUE, "layer %d: kv_from %d has no cache of its own", i, d.kv_from);
        if (o.mixer_kind != d.mixer_kind || o.kv_heads != d.kv_heads || o.dim != d.dim || o.vdim != d.vdim)
            return kr_fail(KR_ERR_VALUE, "layer %d: key / value heads differ from layer %d", i, d.kv_from);
    }
    }      // !ssd1
    if (d.mlp_kind == KR_SERVE_MLP_DENSE && d.ff < 1) return kr_fail(KR_ERR_VALUE, "layer %d: ff %d", i, d.ff);
    if (d.mlp_kind == KR_SERVE_MLP_MOE) {
        if (d.experts < 1 || d.top < 1 || d.groups < 1 || d.keep < 1 || d.keep > d.groups || d.experts % d.groups || d.expert_ff < 1)
            return kr_fail(KR_ERR_VALUE, "layer %d: router sizes (experts %d, top %d, groups %d, keep %d)", i, d.experts, d.top, d.groups, d.keep);
        if (d.top > d.keep * (d.experts / d.groups)) return kr_fail(KR_ERR_VALUE, "layer %d: top %d exceeds the experts of %d groups", i, d.top, d.keep);
        if (d.experts > 8192) return kr_fail(KR_ERR_VALUE, "layer %d: %d experts", i, d.experts);
    } else if (d.mlp_kind != KR_SERVE_MLP_NONE && d.mlp_kind != KR_SERVE_MLP_DENSE) return kr_fail(KR_ERR_VALUE, "layer %d: mlp kind %d", i, d.mlp_kind);
    (void)c;
    return KR_OK;
}

struct Timer {       // HIP events around one kernel family when profiling is on
    kr_serve* s; int fam;
    Timer(kr_serve* s_, int f) : s(s_), fam(f) { if (s->prof) (void)hipEventRecord(s->ev0, s->st); }
    ~Timer() {
        if (!s->prof) return;
        (void)hipEventRecord(s->ev1, s->st); (void)hipEventSynchronize(s->ev1);
        float ms = 0; (void)hipEventElapsedTime(&ms, s->ev0, s->ev1); s->prof_ms[fam] += ms;
    }
};
}  // namespace

extern "C" {

int kr_serve_create(int device_ordinal, const kr_serve_config* cfg, const kr_serve_layer* layers, kr_serve** out) {
    if (!cfg || !layers || !out) return kr_fail(KR_ERR_VALUE, "null argument");
    if (cfg->vocab < 1 || cfg->width < 1 || cfg->n_layers < 1) return kr_fail(KR_ERR_VALUE, "vocab / width / layers");
    if (cfg->dtype != KR_SERVE_BF16 && cfg->dtype != KR_SERVE_F32) return kr_fail(KR_ERR_VALUE, "dtype %d", cfg->dtype);
    if (cfg->norm_kind != KR_SERVE_NORM_LAYER && cfg->norm_kind != KR_SERVE_NORM_RMS) return kr_fail(KR_ERR_VALUE, "norm kind %d", cfg->norm_kind);
    if (cfg->max_slots < 1 || cfg->page_tokens < 1 || cfg->pool_tokens < cfg->page_tokens) return kr_fail(KR_ERR_VALUE, "slots / pages");
    if (cfg->block_kind != KR_SERVE_BLOCK_PARALLEL && cfg->block_kind != KR_SERVE_BLOCK_SEQUENTIAL) return kr_fail(KR_ERR_VALUE, "block kind %d", cfg->block_kind);
    if (cfg->post_norm && cfg->block_kind != KR_SERVE_BLOCK_SEQUENTIAL) return kr_fail(KR_ERR_VALUE, "norms on sublayer outputs need a sequential block");
    if (cfg->norm_groups < 0 || (cfg->norm_groups > 1 && cfg->width % cfg->norm_groups)) return kr_fail(KR_ERR_VALUE, "norm groups %d of width %d", cfg->norm_groups, cfg->width);
    if (cfg->canon_taps < 0 || cfg->canon_taps == 1 || cfg->canon_taps > 64) return kr_fail(KR_ERR_VALUE, "input convolution of %d taps", cfg->canon_taps);
    if ((cfg->canon_taps || cfg->res_gate) && !(cfg->block_kind == KR_SERVE_BLOCK_SEQUENTIAL && cfg->pre_norm && !cfg->post_norm))
        return kr_fail(KR_ERR_VALUE, "input convolution / gated residual need a sequential pre-normed block without output norms");
    if (cfg->embed_norm && !cfg->pre_norm) return kr_fail(KR_ERR_VALUE, "a normed embedding needs pre-normed blocks");
    if (cfg->bigram_buckets < 0) return kr_fail(KR_ERR_VALUE, "bigram buckets %d", cfg->bigram_buckets);
    for (int i = 0; i < cfg->n_layers; i++) { const int rc = check_layer(*cfg, layers, i); if (rc) return rc; }
    int n_dev = 0;
    if (hipGetDeviceCount(&n_dev) != hipSuccess || n_dev <= device_ordinal) return kr_fail(KR_ERR_HIP, "no HIP device %d (the serving store has no CPU path)", device_ordinal);
    KR_HIP(hipSetDevice(device_ordinal));
    kr_serve* s = new kr_serve();
    s->device = device_ordinal; s->c = *cfg; s->f32 = cfg->dtype == KR_SERVE_F32; s->esz = s->f32 ? 4 : 2;
    if (hipStreamCreateWithFlags(&s->st, hipStreamNonBlocking) != hipSuccess) { delete s; return kr_fail(KR_ERR_HIP, "hipStreamCreate failed"); }
    (void)hipEventCreate(&s->ev0); (void)hipEventCreate(&s->ev1);
    s->n_pages = cfg->pool_tokens / cfg->page_tokens;
    for (int p = s->n_pages - 1; p >= 0; p--) s->free_pages.push_back(p);     // pop_back hands out ascending pages first
    s->slots.resize(cfg->max_slots);
    s->h_table.assign((size_t)cfg->max_slots * s->n_pages, 0);
    s->L.resize(cfg->n_layers);
    for (int i = 0; i < cfg->n_layers; i++) {
        SvLayer& l = s->L[i]; l.d = layers[i];
        const kr_serve_layer& d = l.d;
        l.have.assign(KR_SV_N_ROLES, 0);
        l.wsrc = d.weights_of ? d.weights_of - 1 : i;
        l.n_qkv = l.ssd_alone() ? 0 : l.latent() ? d.q_rank + d.kv_rank + d.rot_dims : d.heads * d.dim + (d.kv_from < 0 ? d.kv_heads * (d.dim + (d.v_from_k ? 0 : d.vdim)) : 0);
        l.off_ogate = l.n_qkv;
        if (l.recurrent()) l.n_qkv += d.heads * d.vdim; else if (d.out_gate == KR_SERVE_OGATE_HEAD_SIGMOID) l.n_qkv += d.heads; else if (d.out_gate) l.n_qkv += d.heads * d.vdim;
        l.off_if = l.n_qkv;
        if (d.mixer_kind == KR_SERVE_MIX_MLSTM) l.n_qkv += 2 * d.heads;
        l.off_ssd = l.n_qkv;
        if (l.has_ssd()) l.n_qkv += l.ssd_in_rows();
        l.n_router = d.mlp_kind == KR_SERVE_MLP_MOE ? d.experts * (s->f32 ? 1 : 2) : 0;
        l.n_gu = d.mlp_kind == KR_SERVE_MLP_DENSE ? (l.ungated_ff() ? 1 : 2) * d.ff : (d.mlp_kind == KR_SERVE_MLP_MOE ? 2 * d.shared_ff : 0);
        l.off_router = l.n_qkv; l.off_gu = l.off_router + l.n_router; l.off_rg2 = l.off_gu + l.n_gu;
        l.n_h = l.off_rg2 + ((cfg->res_gate && d.mlp_kind != KR_SERVE_MLP_NONE) ? cfg->width : 0);
        if (d.mlp_kind == KR_SERVE_MLP_MOE) { l.eg.assign(d.experts, 0); l.eu.assign(d.experts, 0); l.ed.assign(d.experts, 0); }
        if (d.rot_dims > 0) {
            const bool parts = d.rot_scaling != KR_SERVE_ROT_LINEAR;       // original / fast / slow take part
            int id = -1;
            for (size_t r = 0; r < s->ropes.size(); r++) {
                const SvRope& q = s->ropes[r];
                if (q.dims == d.rot_dims && q.base == d.rot_base && q.factor == d.rot_factor && q.scaling == d.rot_scaling &&
                    (!parts || (q.original == d.rot_original && q.fast == d.rot_fast && q.slow == d.rot_slow))) id = (int)r;
            }
            if (id < 0) {
                s->ropes.emplace_back(); SvRope& r = s->ropes.back(); r.dims = d.rot_dims; r.base = d.rot_base; r.factor = d.rot_factor; r.scaling = d.rot_scaling;
                r.original = d.rot_original; r.fast = d.rot_fast; r.slow = d.rot_slow; r.mult = 1.0f;
                std::vector<double> f(d.rot_dims / 2);
                if (!parts) {
                    for (int k = 0; k < d.rot_dims / 2; k++) f[k] = std::pow(d.rot_base, -2.0 * k / d.rot_dims) / d.rot_factor;
                } else if (d.rot_scaling == KR_SERVE_ROT_BANDS) {
                    // by wavelength: short ones keep their frequency, long ones are divided by the factor, a linear blend in between
                    for (int k = 0; k < d.rot_dims / 2; k++) {
                        const double fk = std::pow(d.rot_base, -2.0 * k / d.rot_dims), wl = 2.0 * M_PI / fk;
                        if (wl < d.rot_original / d.rot_fast) f[k] = fk;
                        else if (wl > d.rot_original / d.rot_slow) f[k] = fk / d.rot_factor;
                        else { const double sm = (d.rot_original / wl - d.rot_slow) / (d.rot_fast - d.rot_slow); f[k] = (1.0 - sm) * fk / d.rot_factor + sm * fk; }
                    }
                } else {
                    // pair index at which `turns` whole turns fit into `original` positions; pairs below lo keep their frequency, pairs above hi are divided
                    // by the factor, a linear blend between; cos and sin are stretched by 0.1 ln(factor) + 1
                    auto pair_of = [&](double turns) { return d.rot_dims * std::log(d.rot_original / (2.0 * M_PI * turns)) / (2.0 * std::log(d.rot_base)); };
                    const double lo = std::max(std::floor(pair_of(d.rot_fast)), 0.0), hi = std::min(std::ceil(pair_of(d.rot_slow)), (double)(d.rot_dims - 1));
                    for (int k = 0; k < d.rot_dims / 2; k++) {
                        const double fk = std::pow(d.rot_base, -2.0 * k / d.rot_dims);
                        const double ramp = std::min(std::max((k - lo) / std::max(hi - lo, 0.001), 0.0), 1.0);
                        f[k] = fk / d.rot_factor * ramp + fk * (1.0 - ramp);
                    }
                    r.mult = (float)(0.1 * std::log(d.rot_factor) + 1.0);
                }
                if (r.inv_freq.ensure(f.size() * 8) || hipMemcpy(r.inv_freq.p, f.data(), f.size() * 8, hipMemcpyHostToDevice) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "rope table"); }
                id = (int)s->ropes.size() - 1;
            }
            l.rope_id = id;
        }
        if (d.dist_bias) {
            std::vector<float> sl(d.heads);
            for (int h = 0; h < d.heads; h++) sl[h] = (float)std::exp2(-(double)d.dist_bias_exp * (h + 1) / d.heads);
            if (l.slopes.ensure(sl.size() * 4) || hipMemcpy(l.slopes.p, sl.data(), sl.size() * 4, hipMemcpyHostToDevice) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "slopes"); }
        }
        if (d.has_sink == KR_SERVE_SINK_ZERO) {
            if (l.sink.ensure((size_t)d.heads * 4) || hipMemset(l.sink.p, 0, (size_t)d.heads * 4) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "sink"); }
        }
        if (cfg->canon_taps > 1) {
            const size_t b = (size_t)cfg->max_slots * (cfg->canon_taps - 1) * cfg->width * 4;
            if (l.canon_state.ensure(b) || hipMemset(l.canon_state.p, 0, b) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "input convolution state"); }
        }
        if (d.proj_conv > 1) {
            const size_t b = (size_t)cfg->max_slots * (d.proj_conv - 1) * l.pconv_c() * 4;
            if (l.pconv_state.ensure(b) || hipMemset(l.pconv_state.p, 0, b) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "projection convolution state"); }
        }
        if (d.proj_conv && d.proj_bias && !d.weights_of) {       // the biases of q | k | v as one vector: they join the convolution's input
            const size_t b = (size_t)l.pconv_c() * 4;
            if (l.pconv_bias.ensure(b) || hipMemset(l.pconv_bias.p, 0, b) != hipSuccess) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "projection biases"); }
        }
        if (l.has_ssd()) {
            l.ssd_state_stride = (size_t)d.ssd_heads * d.ssd_vdim * d.ssd_state;
            const size_t sb = l.ssd_state_stride * cfg->max_slots * 4, cb = (size_t)cfg->max_slots * (d.ssd_conv - 1) * l.ssd_conv_c() * 4;
            if (l.ssd_state.ensure(sb) || hipMemset(l.ssd_state.p, 0, sb) != hipSuccess || (cb && (l.sconv_state.ensure(cb) || hipMemset(l.sconv_state.p, 0, cb) != hipSuccess))) {
                kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "state-space state of %zu bytes", sb + cb);
            }
        }
        if (l.recurrent()) {
            l.lin_state_stride = (size_t)d.heads * d.vdim * d.dim; l.lin_nm_stride = (size_t)d.heads * ((d.vdim + 15) / 16) * (d.dim + 4);
            const size_t sb = l.lin_state_stride * cfg->max_slots * 4, nb = l.lin_nm_stride * cfg->max_slots * 4;
            if (l.lin_state.ensure(sb) || l.lin_nm.ensure(nb) || hipMemset(l.lin_state.p, 0, sb) != hipSuccess || hipMemset(l.lin_nm.p, 0, nb) != hipSuccess) {
                kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "recurrent state of %zu bytes", sb + nb);
            }
        }
        if (l.has_cache()) {
            const size_t rows = (size_t)s->n_pages * cfg->page_tokens;
            const size_t kb = rows * l.att_heads_kv() * l.att_dim() * s->esz, vb = l.latent() ? 0 : rows * d.kv_heads * d.vdim * s->esz;     // a latent's values are its key rows
            if (l.kpool.ensure(kb) || (vb && l.vpool.ensure(vb))) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "cache pool of %zu bytes", kb + vb); }
            (void)hipMemset(l.kpool.p, 0, kb); if (vb) (void)hipMemset(l.vpool.p, 0, vb);
        }
    }
    if (s->page_table.ensure(s->h_table.size() * 4)) { kr_serve_destroy(s); return kr_fail(KR_ERR_HIP, "page table"); }
    *out = s;
    return KR_OK;
}

void kr_serve_destroy(kr_serve* s) {
    if (!s) return;
    (void)hipSetDevice(s->device);
    if (s->st) { (void)hipStreamSynchronize(s->st); (void)hipStreamDestroy(s->st); }
    if (s->ev0) (void)hipEventDestroy(s->ev0);
    if (s->ev1) (void)hipEventDestroy(s->ev1);
    if (s->h_meta) (void)hipHostFree(s->h_meta);
    for (auto& g : s->graphs) (void)hipGraphExecDestroy(g.exec);
    delete s;
}

int kr_serve_set_tensor(kr_serve* s, int layer, int role, int index, const void* host, int src_dtype, int rows, int cols) {
    if (!s || !host) return kr_fail(KR_ERR_VALUE, "null argument");
    if (src_dtype != KR_SERVE_BF16 && src_dtype != KR_SERVE_F32) return kr_fail(KR_ERR_VALUE, "source dtype %d", src_dtype);
    KR_HIP(hipSetDevice(s->device));
    const int W = s->c.width, V = s->c.vocab;
    const size_t n = (size_t)rows * cols;
#define SHAPE(R_, C_) if (rows != (R_) || cols != (C_)) return kr_fail(KR_ERR_VALUE, "layer %d role %d: shape [%d, %d], expected [%d, %d]", layer, role, rows, cols, (int)(R_), (int)(C_))
    if (layer < 0) {
        switch (role) {
        case KR_SV_EMBED: SHAPE(V, W); s->have_embed = true; return upload(s, s->embed, n, 0, host, src_dtype, n, false);
        case KR_SV_HEAD: SHAPE(V, W); s->have_head = true; return upload(s, s->head, n, 0, host, src_dtype, n, false);
        case KR_SV_FINAL_NORM_W: SHAPE(1, W); s->have_fw = true; return upload_norm_w(s, s->fnorm_w, host, src_dtype, n);
        case KR_SV_EMBED_NORM: if (!s->c.embed_norm) return kr_fail(KR_ERR_VALUE, "the design does not norm its embedding");
            SHAPE(1, W); s->have_enorm = true; return upload_norm_w(s, s->enorm_w, host, src_dtype, n);
        case KR_SV_BIGRAM: if (s->c.bigram_buckets < 1) return kr_fail(KR_ERR_VALUE, "the design has no pair embedding");
            SHAPE(s->c.bigram_buckets + 1, W); s->have_bigram = true; return upload(s, s->bigram, n, 0, host, src_dtype, n, false);
        case KR_SV_FINAL_NORM_B: SHAPE(1, W); s->have_fb = true; return upload(s, s->fnorm_b, n, 0, host, src_dtype, n, true);
        default: return kr_fail(KR_ERR_VALUE, "role %d is not a model-level tensor", role);
        }
    }
    if (layer >= s->c.n_layers) return kr_fail(KR_ERR_VALUE, "layer %d of %d", layer, s->c.n_layers);
    SvLayer& l = s->L[layer]; const kr_serve_layer& d = l.d;
    const int nq = d.heads * d.dim, nk = d.kv_heads * d.dim, nv = d.kv_heads * d.vdim;
    if (role < 0 || role >= KR_SV_N_ROLES) return kr_fail(KR_ERR_VALUE, "role %d", role);
    const bool moe = d.mlp_kind == KR_SERVE_MLP_MOE;
    const bool lat = l.latent();
    if (lat && (role == KR_SV_Q || role == KR_SV_K || role == KR_SV_V)) return kr_fail(KR_ERR_VALUE, "layer %d has a latent mixer", layer);
    if (!lat && role >= KR_SV_DQ && role <= KR_SV_UV) return kr_fail(KR_ERR_VALUE, "layer %d has no latent mixer", layer);
    const bool rec = l.recurrent();
    int rc = KR_OK;
    if (l.wsrc != layer && role != KR_SV_PRE_ADD) return kr_fail(KR_ERR_VALUE, "layer %d uses the tensors of layer %d", layer, l.wsrc);
    const int inner = l.ssd_inner(), sgn = d.ssd_groups * d.ssd_state;
    if (role >= KR_SV_SSD_IN && role <= KR_SV_SSD_O && !l.has_ssd()) return kr_fail(KR_ERR_VALUE, "layer %d has no state-space mixer", layer);
    if (role >= KR_SV_DECAY_A1 && role <= KR_SV_DECAY_A2_B && !l.gla()) return kr_fail(KR_ERR_VALUE, "layer %d has no gla mixer", layer);
    if (l.ssd_alone() && (role == KR_SV_Q || role == KR_SV_K || role == KR_SV_V || role == KR_SV_O)) return kr_fail(KR_ERR_VALUE, "layer %d has a state-space mixer only", layer);
    switch (role) {
    case KR_SV_PRE_ADD:
        if (!d.pre_add) return kr_fail(KR_ERR_VALUE, "layer %d takes no vector before it", layer);
        SHAPE(1, W); rc = upload(s, l.pre_add, n, 0, host, src_dtype, n, true); break;
    case KR_SV_V_BIAS:
        if (d.proj_bias != 2) return kr_fail(KR_ERR_VALUE, "layer %d has no value bias", layer);
        SHAPE(1, nv);
        rc = upload(s, l.v_bias, n, 0, host, src_dtype, n, true);
        if (!rc && d.proj_conv) rc = upload(s, l.pconv_bias, l.pconv_c(), (size_t)nq + nk, host, src_dtype, n, true);
        break;
    case KR_SV_Q_CONV: case KR_SV_K_CONV: case KR_SV_V_CONV:
        if (!d.proj_conv) return kr_fail(KR_ERR_VALUE, "layer %d has no convolution on its projections", layer);
        SHAPE(role == KR_SV_Q_CONV ? nq : role == KR_SV_K_CONV ? nk : nv, d.proj_conv);
        rc = upload(s, l.pconv_w, (size_t)l.pconv_c() * d.proj_conv, (size_t)(role == KR_SV_Q_CONV ? 0 : role == KR_SV_K_CONV ? nq : nq + nk) * d.proj_conv, host, src_dtype, n, true); break;
    case KR_SV_DECAY_A1: SHAPE(d.decay_rank, W); rc = upload(s, l.a1, n, 0, host, src_dtype, n, false); break;
    case KR_SV_DECAY_A2: SHAPE(nq, d.decay_rank); rc = upload(s, l.a2, n, 0, host, src_dtype, n, false); break;
    case KR_SV_DECAY_A2_B: SHAPE(1, nq); rc = upload(s, l.a2_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_IN: SHAPE(l.ssd_in_rows(), W); rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)l.off_ssd * W, host, src_dtype, n, false); break;
    case KR_SV_SSD_CONV: SHAPE(inner + 2 * sgn, d.ssd_conv); rc = upload(s, l.sconv_w, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_CONV_B: SHAPE(1, inner + 2 * sgn); rc = upload(s, l.sconv_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_DT_BIAS: SHAPE(1, d.ssd_heads); rc = upload(s, l.dt_bias, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_A_LOG: SHAPE(1, d.ssd_heads); rc = upload(s, l.a_log, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_D: SHAPE(1, d.ssd_heads); rc = upload(s, l.ssd_d, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_NORM: SHAPE(1, inner); rc = upload(s, l.ssd_norm, n, 0, host, src_dtype, n, true); break;
    case KR_SV_SSD_O: SHAPE(W, inner); rc = upload_cols(s, l.o, W, l.o_cols(), l.att_out_cols(), host, src_dtype, inner); break;
    case KR_SV_Q_BIAS: case KR_SV_K_BIAS: case KR_SV_O_BIAS:
        if (!d.proj_bias) return kr_fail(KR_ERR_VALUE, "layer %d has no projection biases", layer);
        SHAPE(1, role == KR_SV_Q_BIAS ? nq : role == KR_SV_K_BIAS ? nk : W);
        rc = upload(s, role == KR_SV_Q_BIAS ? l.q_bias : role == KR_SV_K_BIAS ? l.k_bias : l.o_bias, n, 0, host, src_dtype, n, true);
        if (!rc && d.proj_conv && role != KR_SV_O_BIAS) rc = upload(s, l.pconv_bias, l.pconv_c(), role == KR_SV_Q_BIAS ? 0 : (size_t)nq, host, src_dtype, n, true);
        break;
    case KR_SV_OUT_GATE:
        if (!rec && !d.out_gate) return kr_fail(KR_ERR_VALUE, "layer %d has no output gate", layer);
        SHAPE((rec || d.out_gate == KR_SERVE_OGATE_ELEM_SIGMOID) ? d.heads * d.vdim : d.heads, W); rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)l.off_ogate * W, host, src_dtype, n, false); break;
    case KR_SV_IGATE: case KR_SV_FGATE:
        if (d.mixer_kind != KR_SERVE_MIX_MLSTM) return kr_fail(KR_ERR_VALUE, "layer %d has no input / forget gates", layer);
        SHAPE(d.heads, W); rc = upload(s, l.hw, (size_t)l.n_h * W, ((size_t)l.off_if + (role == KR_SV_FGATE ? d.heads : 0)) * W, host, src_dtype, n, false); break;
    case KR_SV_IGATE_B: case KR_SV_FGATE_B:
        if (d.mixer_kind != KR_SERVE_MIX_MLSTM) return kr_fail(KR_ERR_VALUE, "layer %d has no input / forget gates", layer);
        SHAPE(1, d.heads); rc = upload(s, role == KR_SV_IGATE_B ? l.i_bias : l.f_bias, n, 0, host, src_dtype, n, true); break;
    case KR_SV_LIN_NORM:
        if (!rec || !d.lin_norm_weight) return kr_fail(KR_ERR_VALUE, "layer %d has no weight on its mixer's output norm", layer);
        SHAPE(1, d.lin_norm_weight == 2 ? d.vdim : d.heads * d.vdim); rc = upload(s, l.lin_norm, n, 0, host, src_dtype, n, true); break;
    case KR_SV_LIN_DECAY:
        if (d.mixer_kind != KR_SERVE_MIX_RETENTION) return kr_fail(KR_ERR_VALUE, "layer %d is no retention layer", layer);
        SHAPE(1, d.heads); rc = upload(s, l.decay, n, 0, host, src_dtype, n, true); break;
    case KR_SV_CANON:
        if (s->c.canon_taps < 2) return kr_fail(KR_ERR_VALUE, "the design has no input convolution");
        SHAPE(W, s->c.canon_taps); rc = upload(s, l.canon, n, 0, host, src_dtype, n, true); break;
    case KR_SV_RES_GATE1: case KR_SV_RES_GATE2:
        if (!s->c.res_gate || (role == KR_SV_RES_GATE2 && d.mlp_kind == KR_SERVE_MLP_NONE)) return kr_fail(KR_ERR_VALUE, "layer %d has no such residual gate", layer);
        SHAPE(W, W);
        if (role == KR_SV_RES_GATE1) rc = upload(s, l.rg1, n, 0, host, src_dtype, n, false);
        else rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)l.off_rg2 * W, host, src_dtype, n, false);
        break;
    case KR_SV_RES_GATE1_B: case KR_SV_RES_GATE2_B:
        if (!s->c.res_gate || (role == KR_SV_RES_GATE2_B && d.mlp_kind == KR_SERVE_MLP_NONE)) return kr_fail(KR_ERR_VALUE, "layer %d has no such residual gate", layer);
        SHAPE(1, W); rc = upload(s, role == KR_SV_RES_GATE1_B ? l.rg1_b : l.rg2_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_NORM2_W: SHAPE(1, W); rc = upload_norm_w(s, l.norm2_w, host, src_dtype, n); break;
    case KR_SV_NORM2_B: SHAPE(1, W); rc = upload(s, l.norm2_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_POST1_W: SHAPE(1, W); rc = upload(s, l.post1_w, n, 0, host, src_dtype, n, true); break;
    case KR_SV_POST1_B: SHAPE(1, W); rc = upload(s, l.post1_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_POST2_W: SHAPE(1, W); rc = upload(s, l.post2_w, n, 0, host, src_dtype, n, true); break;
    case KR_SV_POST2_B: SHAPE(1, W); rc = upload(s, l.post2_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_Q_NORM: case KR_SV_K_NORM:
        if (d.qk_unit_norm != KR_SERVE_QKNORM_WEIGHTED && d.qk_unit_norm != KR_SERVE_QKNORM_WHOLE) return kr_fail(KR_ERR_VALUE, "layer %d has no weighted q / k norm", layer);
        SHAPE(1, d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE ? (role == KR_SV_Q_NORM ? nq : nk) : d.dim); rc = upload(s, role == KR_SV_Q_NORM ? l.q_norm : l.k_norm, n, 0, host, src_dtype, n, true); break;
    case KR_SV_VMIX: if (d.v_mix != KR_SERVE_VMIX_BLEND) return kr_fail(KR_ERR_VALUE, "layer %d blends no values", layer);
        SHAPE(1, 1); rc = upload(s, l.vmix, n, 0, host, src_dtype, n, true); break;
    case KR_SV_ROUTER_BIAS: if (!moe || !d.router_bias) return kr_fail(KR_ERR_VALUE, "layer %d has no router bias", layer);
        SHAPE(1, d.experts); rc = upload(s, l.router_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_DQ: SHAPE(d.q_rank, W); rc = upload(s, l.hw, (size_t)l.n_h * W, 0, host, src_dtype, n, false); break;
    case KR_SV_DKV: SHAPE(d.kv_rank + d.rot_dims, W); rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)d.q_rank * W, host, src_dtype, n, false); break;
    case KR_SV_DQ_NORM: SHAPE(1, d.q_rank); rc = upload(s, l.dq_norm, n, 0, host, src_dtype, n, true); break;
    case KR_SV_DKV_NORM: SHAPE(1, d.kv_rank); rc = upload(s, l.dkv_norm, n, 0, host, src_dtype, n, true); break;
    case KR_SV_UQ: SHAPE(d.heads * (d.dim + d.rot_dims), d.q_rank); rc = upload(s, l.uq, n, 0, host, src_dtype, n, false); break;
    case KR_SV_UV: SHAPE(d.heads * d.vdim, d.kv_rank); rc = upload(s, l.uv, n, 0, host, src_dtype, n, false); break;
    case KR_SV_UK: {      // [heads * dim, kv_rank] -> per head [kv_rank, dim]: the matrix that carries a head's plain query part into the latent space
        SHAPE(d.heads * d.dim, d.kv_rank);
        std::vector<float> tr(n);
        for (int h = 0; h < d.heads; h++)
            for (int e = 0; e < d.dim; e++)
                for (int r = 0; r < d.kv_rank; r++) {
                    const size_t src = ((size_t)h * d.dim + e) * d.kv_rank + r;
                    tr[((size_t)h * d.kv_rank + r) * d.dim + e] = src_dtype == KR_SERVE_F32 ? ((const float*)host)[src] : bf16_to_f32_host(((const uint16_t*)host)[src]);
                }
        rc = upload(s, l.ukT, n, 0, tr.data(), KR_SERVE_F32, n, false); break;
    }
    case KR_SV_NORM_W: SHAPE(1, W); rc = upload_norm_w(s, l.norm_w, host, src_dtype, n); break;
    case KR_SV_NORM_B: SHAPE(1, W); rc = upload(s, l.norm_b, n, 0, host, src_dtype, n, true); break;
    case KR_SV_Q: SHAPE(nq, W); rc = upload(s, l.hw, (size_t)l.n_h * W, 0, host, src_dtype, n, false); break;
    case KR_SV_K: if (d.kv_from >= 0) return kr_fail(KR_ERR_VALUE, "layer %d borrows its keys", layer);
        SHAPE(nk, W); rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)nq * W, host, src_dtype, n, false); break;
    case KR_SV_V: if (d.kv_from >= 0 || d.v_from_k) return kr_fail(KR_ERR_VALUE, "layer %d has no value projection", layer);
        SHAPE(nv, W); rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)(nq + nk) * W, host, src_dtype, n, false); break;
    case KR_SV_O: SHAPE(W, d.heads * d.vdim);
        if (l.has_ssd()) rc = upload_cols(s, l.o, W, l.o_cols(), 0, host, src_dtype, d.heads * d.vdim);
        else rc = upload(s, l.o, n, 0, host, src_dtype, n, false);
        break;
    case KR_SV_SINK: if (d.has_sink != KR_SERVE_SINK_TENSOR) return kr_fail(KR_ERR_VALUE, "layer %d has no sink tensor", layer);
        SHAPE(1, d.heads); rc = upload(s, l.sink, n, 0, host, src_dtype, n, true); break;
    case KR_SV_GATE: case KR_SV_UP:
        if (d.mlp_kind != KR_SERVE_MLP_DENSE || (role == KR_SV_GATE && l.ungated_ff())) return kr_fail(KR_ERR_VALUE, "layer %d has no such dense feed-forward tensor", layer);
        SHAPE(d.ff, W); rc = upload(s, l.hw, (size_t)l.n_h * W, ((size_t)l.off_gu + ((role == KR_SV_UP && !l.ungated_ff()) ? d.ff : 0)) * W, host, src_dtype, n, false); break;
    case KR_SV_DOWN:
        if (d.mlp_kind != KR_SERVE_MLP_DENSE) return kr_fail(KR_ERR_VALUE, "layer %d has no dense feed-forward", layer);
        SHAPE(W, d.ff); rc = upload(s, l.down, n, 0, host, src_dtype, n, false); break;
    case KR_SV_ROUTER: {
        if (!moe) return kr_fail(KR_ERR_VALUE, "layer %d has no router", layer);
        SHAPE(d.experts, W);
        if (s->f32) { rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)l.off_router * W, host, src_dtype, n, false); break; }
        // bf16 store: gate = hi + lo, both bf16, rows [0, E) and [E, 2E) of one matrix
        std::vector<uint16_t> hl(2 * n);
        for (size_t k = 0; k < n; k++) {
            const float g = src_dtype == KR_SERVE_F32 ? ((const float*)host)[k] : bf16_to_f32_host(((const uint16_t*)host)[k]);
            hl[k] = f32_to_bf16_host(g); hl[n + k] = f32_to_bf16_host(g - bf16_to_f32_host(hl[k]));
        }
        rc = upload(s, l.hw, (size_t)l.n_h * W, (size_t)l.off_router * W, hl.data(), KR_SERVE_BF16, 2 * n, false); break;
    }
    case KR_SV_EXPERT_GATE: case KR_SV_EXPERT_UP: case KR_SV_EXPERT_DOWN: {
        if (!moe) return kr_fail(KR_ERR_VALUE, "layer %d has no experts", layer);
        if (index < 0 || index >= d.experts) return kr_fail(KR_ERR_VALUE, "expert %d of %d", index, d.experts);
        const int F = d.expert_ff;
        if (role == KR_SV_EXPERT_DOWN) { SHAPE(W, F); rc = upload(s, l.edown, (size_t)d.experts * W * F, (size_t)index * W * F, host, src_dtype, n, false); l.ed[index] = 1; }
        else {
            SHAPE(F, W);
            rc = upload(s, l.egu, (size_t)d.experts * 2 * F * W, (size_t)index * 2 * F * W + (role == KR_SV_EXPERT_UP ? (size_t)F * W : 0), host, src_dtype, n, false);
            (role == KR_SV_EXPERT_UP ? l.eu : l.eg)[index] = 1;
        }
        break;
    }
    case KR_SV_SHARED_GATE: case KR_SV_SHARED_UP:
        if (!moe || d.shared_ff < 1) return kr_fail(KR_ERR_VALUE, "layer %d has no shared expert", layer);
        SHAPE(d.shared_ff, W); rc = upload(s, l.hw, (size_t)l.n_h * W, ((size_t)l.off_gu + (role == KR_SV_SHARED_UP ? d.shared_ff : 0)) * W, host, src_dtype, n, false); break;
    case KR_SV_SHARED_DOWN:
        if (!moe || d.shared_ff < 1) return kr_fail(KR_ERR_VALUE, "layer %d has no shared expert", layer);
        SHAPE(W, d.shared_ff); rc = upload(s, l.sdown, n, 0, host, src_dtype, n, false); break;
    default: return kr_fail(KR_ERR_VALUE, "role %d is not a layer tensor", role);
    }
#undef SHAPE
    if (rc == KR_OK) l.have[role] = 1;
    return rc;
}

int kr_serve_fill_synthetic(kr_serve* s, uint64_t seed, float amp) {
    if (!s) return kr_fail(KR_ERR_VALUE, "null argument");
    KR_HIP(hipSetDevice(s->device));
    const int W = s->c.width, V = s->c.vocab;
    uint64_t k = seed;
    // storage-type matrix [n] with fan-in `in`; f32 vectors of ones (`one`) or zeros
    auto mat = [&](DevBuf& b, size_t n, int in) -> int {
        if (!b.p) { if (b.ensure(n * s->esz)) return 1; s->weight_bytes += n * s->esz; }
        kr_sv_fill_uniform(b.p, s->f32, n, ++k, amp / std::sqrt((float)in), s->st); return 0;
    };
    auto vec = [&](DevBuf& b, size_t n, bool one) -> int {
        if (!b.p) { if (b.ensure(n * 4)) return 1; s->weight_bytes += n * 4; }
        std::vector<float> h(n, one ? 1.0f : 0.0f);
        return hipMemcpy(b.p, h.data(), n * 4, hipMemcpyHostToDevice) != hipSuccess;
    };
    const bool nb = s->c.norm_bias != 0;
    int bad = mat(s->embed, (size_t)V * W, 1) | mat(s->head, (size_t)V * W, W) | vec(s->fnorm_w, W, true) | (nb ? vec(s->fnorm_b, W, false) : 0);
    s->have_embed = s->have_head = s->have_fw = s->have_fb = true;
    if (s->c.embed_norm) { bad |= vec(s->enorm_w, W, true); s->have_enorm = true; }
    if (s->c.bigram_buckets > 0) { bad |= mat(s->bigram, (size_t)(s->c.bigram_buckets + 1) * W, 1); s->have_bigram = true; }
    // a vector of n f32 values uniform in +-amp_v around mid
    auto vecu = [&](DevBuf& b, size_t n, float mid, float amp_v) -> int {
        if (vec(b, n, false)) return 1;
        kr_sv_fill_uniform(b.p, true, n, ++k, amp_v, s->st);
        if (mid != 0.0f) {
            if (hipStreamSynchronize(s->st) != hipSuccess) return 1;
            std::vector<float> h(n);
            if (hipMemcpy(h.data(), b.p, n * 4, hipMemcpyDeviceToHost) != hipSuccess) return 1;
            for (float& v : h) v += mid;
            return hipMemcpy(b.p, h.data(), n * 4, hipMemcpyHostToDevice) != hipSuccess;
        }
        return 0;
    };
    for (SvLayer& l : s->L) {
        const kr_serve_layer& d = l.d;
        if (d.pre_add) bad |= vecu(l.pre_add, W, 0.0f, 0.1f);
        if (l.wsrc != (int)(&l - s->L.data())) { std::fill(l.have.begin(), l.have.end(), 1); continue; }      // the tensors are another layer's
        bad |= mat(l.hw, (size_t)l.n_h * W, W) | mat(l.o, (size_t)W * l.o_cols(), l.o_cols());
        if (d.proj_bias == 2) bad |= vec(l.v_bias, (size_t)d.kv_heads * d.vdim, false);
        if (d.proj_conv) {           // taps of about 1 / taps: the convolved projection stays at the projection's scale
            bad |= vecu(l.pconv_w, (size_t)l.pconv_c() * d.proj_conv, 1.0f / (float)d.proj_conv, 0.5f / (float)d.proj_conv);
        }
        if (l.gla()) bad |= mat(l.a1, (size_t)d.decay_rank * W, W) | mat(l.a2, (size_t)d.heads * d.dim * d.decay_rank, d.decay_rank) | vecu(l.a2_b, (size_t)d.heads * d.dim, 3.0f, 1.0f);
        if (l.has_ssd()) {
            bad |= vecu(l.sconv_w, (size_t)l.ssd_conv_c() * d.ssd_conv, 1.0f / (float)d.ssd_conv, 0.5f / (float)d.ssd_conv) | vec(l.sconv_b, l.ssd_conv_c(), false) |
                   vecu(l.dt_bias, d.ssd_heads, -2.0f, 1.0f) | vecu(l.a_log, d.ssd_heads, 0.0f, 1.0f) | vec(l.ssd_d, d.ssd_heads, true) | vec(l.ssd_norm, l.ssd_inner(), true);
        }
        if (s->c.pre_norm) bad |= vec(l.norm_w, W, true) | (nb ? vec(l.norm_b, W, false) : 0);
        if (s->c.pre_norm && s->c.block_kind == KR_SERVE_BLOCK_SEQUENTIAL) bad |= vec(l.norm2_w, W, true) | (nb ? vec(l.norm2_b, W, false) : 0);
        if (s->c.post_norm) bad |= vec(l.post1_w, W, true) | vec(l.post2_w, W, true) | (nb ? vec(l.post1_b, W, false) | vec(l.post2_b, W, false) : 0);
        if (d.has_sink == KR_SERVE_SINK_TENSOR) bad |= vec(l.sink, d.heads, false);
        if (d.qk_unit_norm == KR_SERVE_QKNORM_WEIGHTED) bad |= vec(l.q_norm, d.dim, true) | vec(l.k_norm, d.dim, true);
        if (d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE) bad |= vec(l.q_norm, (size_t)d.heads * d.dim, true) | vec(l.k_norm, (size_t)d.kv_heads * d.dim, true);
        if (d.proj_bias) bad |= vec(l.q_bias, (size_t)d.heads * d.dim, false) | vec(l.k_bias, (size_t)d.kv_heads * d.dim, false) | vec(l.o_bias, W, false);
        if (s->c.canon_taps > 1) {           // taps of 1 / (2 taps): the convolved input stays at the input's scale
            bad |= vec(l.canon, (size_t)W * s->c.canon_taps, true);
            if (!bad) kr_sv_fill_uniform(l.canon.p, true, (size_t)W * s->c.canon_taps, ++k, 0.5f / (float)s->c.canon_taps, s->st);
        }
        if (s->c.res_gate) {
            bad |= mat(l.rg1, (size_t)W * W, W) | vec(l.rg1_b, W, false);
            if (d.mlp_kind != KR_SERVE_MLP_NONE) bad |= vec(l.rg2_b, W, false);
        }
        if (l.recurrent()) {
            if (d.lin_norm_weight) bad |= vec(l.lin_norm, d.lin_norm_weight == 2 ? (size_t)d.vdim : (size_t)d.heads * d.vdim, true);
            if (d.mixer_kind == KR_SERVE_MIX_MLSTM) bad |= vec(l.i_bias, d.heads, false) | vec(l.f_bias, d.heads, true);
            else if (d.mixer_kind == KR_SERVE_MIX_RETENTION) {
                std::vector<float> dc(d.heads);
                for (int h = 0; h < d.heads; h++) dc[h] = 1.0f - std::exp2(-5.0f - (float)(h % 8));
                bad |= vec(l.decay, d.heads, true);
                if (!bad) bad |= hipMemcpy(l.decay.p, dc.data(), dc.size() * 4, hipMemcpyHostToDevice) != hipSuccess;
            }
        }
        if (d.v_mix == KR_SERVE_VMIX_BLEND) { bad |= vec(l.vmix, 1, true); const float half = 0.5f; bad |= hipMemcpy(l.vmix.p, &half, 4, hipMemcpyHostToDevice) != hipSuccess; }
        if (l.latent()) {
            bad |= vec(l.dq_norm, d.q_rank, true) | vec(l.dkv_norm, d.kv_rank, true) | mat(l.uq, (size_t)d.heads * (d.dim + d.rot_dims) * d.q_rank, d.q_rank) |
                   mat(l.ukT, (size_t)d.heads * d.kv_rank * d.dim, d.kv_rank) | mat(l.uv, (size_t)d.heads * d.vdim * d.kv_rank, d.kv_rank);
        }
        if (d.mlp_kind == KR_SERVE_MLP_DENSE) bad |= mat(l.down, (size_t)W * d.ff, d.ff);
        if (d.mlp_kind == KR_SERVE_MLP_MOE) {
            if (!s->f32 && l.hw.p) kr_sv_fill_uniform((uint16_t*)l.hw.p + ((size_t)l.off_router + d.experts) * W, false, (size_t)d.experts * W, 0, 0.0f, s->st);   // the gate's lo rows: zero
            if (d.router_bias) bad |= vec(l.router_b, d.experts, false);
            bad |= mat(l.egu, (size_t)d.experts * 2 * d.expert_ff * W, W) | mat(l.edown, (size_t)d.experts * W * d.expert_ff, d.expert_ff);
            if (d.shared_ff > 0) bad |= mat(l.sdown, (size_t)W * d.shared_ff, d.shared_ff);
            std::fill(l.eg.begin(), l.eg.end(), 1); std::fill(l.eu.begin(), l.eu.end(), 1); std::fill(l.ed.begin(), l.ed.end(), 1);
        }
        std::fill(l.have.begin(), l.have.end(), 1);
    }
    if (bad) return kr_fail(KR_ERR_HIP, "synthetic weights: allocation or copy failed");
    KR_HIP(hipStreamSynchronize(s->st));
    return KR_OK;
}

int kr_serve_finalize(kr_serve* s) {
    if (!s) return kr_fail(KR_ERR_VALUE, "null argument");
    if (!s->have_embed || !s->have_head || !s->have_fw) return kr_fail(KR_ERR_STATE, "embedding, head or final norm missing");
    if (s->c.norm_bias && !s->have_fb) return kr_fail(KR_ERR_STATE, "final norm bias missing");
    if (s->c.embed_norm && !s->have_enorm) return kr_fail(KR_ERR_STATE, "embedding norm missing");
    if (s->c.bigram_buckets > 0 && !s->have_bigram) return kr_fail(KR_ERR_STATE, "pair embedding missing");
    const bool seq = s->c.block_kind == KR_SERVE_BLOCK_SEQUENTIAL, nb = s->c.norm_bias != 0;
    for (int i = 0; i < s->c.n_layers; i++) {
        SvLayer& l = s->L[i]; const kr_serve_layer& d = l.d;
        const bool has_ff = d.mlp_kind != KR_SERVE_MLP_NONE;
        if (d.pre_add && !l.have[KR_SV_PRE_ADD]) return kr_fail(KR_ERR_STATE, "layer %d: the vector before the layer is missing", i);
        if (l.wsrc != i) continue;
        std::vector<int> need;
        if (!l.ssd_alone()) need.push_back(KR_SV_O);
        if (s->c.pre_norm) { need.push_back(KR_SV_NORM_W); if (nb) need.push_back(KR_SV_NORM_B); }
        if (s->c.pre_norm && seq && has_ff) { need.push_back(KR_SV_NORM2_W); if (nb) need.push_back(KR_SV_NORM2_B); }
        if (s->c.post_norm) { need.push_back(KR_SV_POST1_W); if (nb) need.push_back(KR_SV_POST1_B); }
        if (s->c.post_norm && has_ff) { need.push_back(KR_SV_POST2_W); if (nb) need.push_back(KR_SV_POST2_B); }
        if (l.latent()) for (int r : {KR_SV_DQ, KR_SV_DQ_NORM, KR_SV_UQ, KR_SV_DKV, KR_SV_DKV_NORM, KR_SV_UK, KR_SV_UV}) need.push_back(r);
        else if (!l.ssd_alone()) {
            need.push_back(KR_SV_Q);
            if (d.kv_from < 0) { need.push_back(KR_SV_K); if (!d.v_from_k) need.push_back(KR_SV_V); }
        }
        if (d.qk_unit_norm == KR_SERVE_QKNORM_WEIGHTED || d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE) { need.push_back(KR_SV_Q_NORM); if (d.kv_from < 0) need.push_back(KR_SV_K_NORM); }
        if (d.proj_bias) { need.push_back(KR_SV_Q_BIAS); need.push_back(KR_SV_O_BIAS); if (d.kv_from < 0) need.push_back(KR_SV_K_BIAS); }
        if (d.proj_bias == 2) need.push_back(KR_SV_V_BIAS);
        if (d.proj_conv) for (int r : {KR_SV_Q_CONV, KR_SV_K_CONV, KR_SV_V_CONV}) need.push_back(r);
        if (l.gla()) for (int r : {KR_SV_DECAY_A1, KR_SV_DECAY_A2, KR_SV_DECAY_A2_B}) need.push_back(r);
        if (l.has_ssd()) for (int r = KR_SV_SSD_IN; r <= KR_SV_SSD_O; r++) need.push_back(r);
        if (d.out_gate || l.recurrent()) need.push_back(KR_SV_OUT_GATE);
        if (l.recurrent() && d.lin_norm_weight) need.push_back(KR_SV_LIN_NORM);
        if (d.mixer_kind == KR_SERVE_MIX_RETENTION) need.push_back(KR_SV_LIN_DECAY);
        if (d.mixer_kind == KR_SERVE_MIX_MLSTM) for (int r : {KR_SV_IGATE, KR_SV_IGATE_B, KR_SV_FGATE, KR_SV_FGATE_B}) need.push_back(r);
        if (s->c.canon_taps > 1) need.push_back(KR_SV_CANON);
        if (s->c.res_gate) { need.push_back(KR_SV_RES_GATE1); need.push_back(KR_SV_RES_GATE1_B); if (has_ff) { need.push_back(KR_SV_RES_GATE2); need.push_back(KR_SV_RES_GATE2_B); } }
        if (d.v_mix == KR_SERVE_VMIX_BLEND) need.push_back(KR_SV_VMIX);
        if (d.has_sink == KR_SERVE_SINK_TENSOR) need.push_back(KR_SV_SINK);
        if (d.mlp_kind == KR_SERVE_MLP_DENSE) { if (!l.ungated_ff()) need.push_back(KR_SV_GATE); need.push_back(KR_SV_UP); need.push_back(KR_SV_DOWN); }
        if (d.mlp_kind == KR_SERVE_MLP_MOE) {
            need.push_back(KR_SV_ROUTER);
            if (d.router_bias) need.push_back(KR_SV_ROUTER_BIAS);
            if (d.shared_ff > 0) { need.push_back(KR_SV_SHARED_GATE); need.push_back(KR_SV_SHARED_UP); need.push_back(KR_SV_SHARED_DOWN); }
            for (int e = 0; e < d.experts; e++) if (!l.eg[e] || !l.eu[e] || !l.ed[e]) return kr_fail(KR_ERR_STATE, "layer %d: expert %d incomplete", i, e);
        }
        for (int r : need) if (!l.have[r]) return kr_fail(KR_ERR_STATE, "layer %d: tensor of role %d missing", i, r);
    }
    s->finalized = true;
    return KR_OK;
}

int kr_serve_abi(void) { return KR_SERVE_ABI; }

int kr_serve_admit(kr_serve* s, int* slot_out) {
    if (!s || !slot_out) return kr_fail(KR_ERR_VALUE, "null argument");
    for (size_t i = 0; i < s->slots.size(); i++) if (!s->slots[i].live) { s->slots[i].live = true; s->slots[i].len = 0; s->slots[i].last_token = -1; *slot_out = (int)i; return KR_OK; }
    return kr_fail(KR_ERR_STATE, "all %zu request slots are live", s->slots.size());
}

int kr_serve_release(kr_serve* s, int slot) {
    if (!s || slot < 0 || slot >= (int)s->slots.size() || !s->slots[slot].live) return kr_fail(KR_ERR_VALUE, "slot %d is not live", slot);
    SvSlot& sl = s->slots[slot];
    for (size_t i = sl.pages.size(); i-- > 0;) s->free_pages.push_back(sl.pages[i]);
    sl.pages.clear(); sl.len = 0; sl.live = false;
    return KR_OK;
}

int kr_serve_slot_len(kr_serve* s, int slot, int* len_out) {
    if (!s || !len_out || slot < 0 || slot >= (int)s->slots.size() || !s->slots[slot].live) return kr_fail(KR_ERR_VALUE, "slot %d is not live", slot);
    *len_out = s->slots[slot].len; return KR_OK;
}
int kr_serve_free_pages(kr_serve* s, int* n_out) { if (!s || !n_out) return kr_fail(KR_ERR_VALUE, "null argument"); *n_out = (int)s->free_pages.size(); return KR_OK; }
size_t kr_serve_device_bytes(const kr_serve* s) {
    if (!s) return 0;
    size_t b = s->weight_bytes;
    for (const SvLayer& l : s->L) b += l.kpool.bytes + l.vpool.bytes;
    return b;
}
int kr_serve_set_capture(kr_serve* s, int enable) { if (!s) return kr_fail(KR_ERR_VALUE, "null argument"); s->capture = enable != 0; s->cap_T = 0; return KR_OK; }
int kr_serve_read_capture(kr_serve* s, float* out_host, size_t n_floats) {
    if (!s || !out_host) return kr_fail(KR_ERR_VALUE, "null argument");
    const size_t have = (size_t)s->c.n_layers * s->cap_T * s->c.width;
    if (n_floats != have) return kr_fail(KR_ERR_VALUE, "capture holds %zu floats", have);
    KR_HIP(hipMemcpy(out_host, s->cap.p, have * 4, hipMemcpyDeviceToHost));
    return KR_OK;
}
int kr_serve_set_profiling(kr_serve* s, int enable) { if (!s) return kr_fail(KR_ERR_VALUE, "null argument"); s->prof = enable != 0; for (double& m : s->prof_ms) m = 0; return KR_OK; }
int kr_serve_get_profile(kr_serve* s, double* ms, int n) { if (!s || !ms) return kr_fail(KR_ERR_VALUE, "null argument"); for (int i = 0; i < n && i < 8; i++) ms[i] = s->prof_ms[i]; return KR_OK; }

int kr_serve_step(kr_serve* s, int n_entries, const int* slots, const int* counts, const int* tokens, int n_want, const int* want_rows, float* logits_out,
                  int* argmax_out) {
    if (!s || !slots || !counts || !tokens || n_entries < 1 || n_want < 0 || (n_want && !want_rows)) return kr_fail(KR_ERR_VALUE, "bad step arguments");
    if (!s->finalized) return kr_fail(KR_ERR_STATE, "the store is not finalized");
    KR_HIP(hipSetDevice(s->device));
    const kr_serve_config& c = s->c;
    const int W = c.width, PT = c.page_tokens;
    // ---- admission checks and pages, before anything changes
    long T64 = 0; int need_pages = 0;
    for (int e = 0; e < n_entries; e++) {
        const int sl = slots[e];
        if (sl < 0 || sl >= c.max_slots || !s->slots[sl].live) return kr_fail(KR_ERR_VALUE, "entry %d: slot %d is not live", e, sl);
        for (int f = 0; f < e; f++) if (slots[f] == sl) return kr_fail(KR_ERR_VALUE, "slot %d appears twice in one step", sl);
        if (counts[e] < 1) return kr_fail(KR_ERR_VALUE, "entry %d: %d tokens", e, counts[e]);
        const SvSlot& q = s->slots[sl];
        need_pages += (q.len + counts[e] + PT - 1) / PT - (int)q.pages.size();
        T64 += counts[e];
    }
    if (T64 > (1 << 24)) return kr_fail(KR_ERR_VALUE, "%ld tokens in one step", T64);
    const int T = (int)T64;
    for (int i = 0; i < T; i++) if (tokens[i] < 0 || tokens[i] >= c.vocab) return kr_fail(KR_ERR_VALUE, "token %d outside the vocabulary", tokens[i]);
    for (int i = 0; i < n_want; i++) if (want_rows[i] < 0 || want_rows[i] >= T) return kr_fail(KR_ERR_VALUE, "wanted row %d of %d", want_rows[i], T);
    if (need_pages > (int)s->free_pages.size()) return kr_fail(KR_ERR_STATE, "cache pool exhausted: %d pages needed, %zu free", need_pages, s->free_pages.size());
    // ---- per-step arrays: tokens | slot | pos | want | page table
    const size_t n_meta = (size_t)4 * T + n_want + 3 * (size_t)n_entries + 2;      // ... | first row of every entry and the end | slot of every entry | first 64-token block of every entry and the end
    const size_t meta_bytes = (n_meta + s->h_table.size()) * 4;
    if (meta_bytes > s->h_meta_bytes) {
        if (s->h_meta) (void)hipHostFree(s->h_meta);
        s->h_meta = nullptr; s->h_meta_bytes = 0;
        KR_HIP(hipHostMalloc(&s->h_meta, meta_bytes * 2, hipHostMallocDefault));
        s->h_meta_bytes = meta_bytes * 2;
    }
    int* hm = (int*)s->h_meta;
    int* h_tok = hm; int* h_slot = hm + T; int* h_pos = hm + 2 * T; int* h_brow = hm + 3 * T; int* h_want = hm + 4 * T; /* h_brow: row of the pair embedding */ int* h_eoff = h_want + n_want; int* h_eslot = h_eoff + n_entries + 1; int* h_echunk = h_eslot + n_entries;
    int* h_tab = hm + n_meta;
    int max_pos = 0, n_chunks = 0, max_count = 0;
    {
        int t = 0;
        for (int e = 0; e < n_entries; e++) {
            SvSlot& q = s->slots[slots[e]];
            max_pos = std::max(max_pos, q.len + counts[e] - 1);
            h_eoff[e] = t; h_eslot[e] = slots[e]; h_echunk[e] = n_chunks; n_chunks += (counts[e] + 63) / 64; max_count = std::max(max_count, counts[e]);
            const int np = (q.len + counts[e] + PT - 1) / PT;
            while ((int)q.pages.size() < np) { q.pages.push_back(s->free_pages.back()); s->free_pages.pop_back(); }
            for (int i = 0; i < counts[e]; i++, t++) {
                h_tok[t] = tokens[t]; h_slot[t] = slots[e]; h_pos[t] = q.len + i;
                const int prev = q.len + i == 0 ? -1 : q.last_token;
                h_brow[t] = c.bigram_buckets > 0 ? (prev < 0 ? c.bigram_buckets : (int)(((long long)prev * c.bigram_mul_prev + (long long)tokens[t] * c.bigram_mul_cur) % c.bigram_buckets)) : 0;
                q.last_token = tokens[t];
            }
            for (size_t p = 0; p < q.pages.size(); p++) s->h_table[(size_t)slots[e] * s->n_pages + p] = q.pages[p];
            q.len += counts[e];
        }
        h_eoff[n_entries] = t; h_echunk[n_entries] = n_chunks;
        for (int i = 0; i < n_want; i++) h_want[i] = want_rows[i];
        std::memcpy(h_tab, s->h_table.data(), s->h_table.size() * 4);
    }
    if (s->meta.ensure(meta_bytes)) return kr_fail(KR_ERR_HIP, "step arrays");
    hipStream_t st = s->st;
    KR_HIP(hipMemcpyAsync(s->meta.p, hm, meta_bytes, hipMemcpyHostToDevice, st));
    const int* d_tok = (const int*)s->meta.p; const int* d_slot = d_tok + T; const int* d_pos = d_tok + 2 * T; const int* d_brow = d_tok + 3 * T; const int* d_want = d_tok + 4 * T;
    const int* d_eoff = d_want + n_want; const int* d_eslot = d_eoff + n_entries + 1; const int* d_echunk = d_eslot + n_entries;
    const int* d_tab = d_tok + n_meta;
    // ---- scratch sized for this step
    const bool seq = c.block_kind == KR_SERVE_BLOCK_SEQUENTIAL;
    size_t max_qkv = 0, max_att = 0, max_gu = 0, max_y = 0, max_rows = 0, max_pairs = 0, max_vf = 0; int max_E = 1;
    size_t lq_c = 0, lq_2 = 0, lq_n = 0, lq_e = 0, att2 = 0, head_i = 0, max_lin = 0, lin_tok = 0, lin_sb = 0, lin_nb = 0; bool whole_norm = false;
    size_t max_pconv = 0, max_sconv = 0, max_ga1 = 0, max_gz = 0, max_ssdz = 0;
    // prompt portions take the chunked form of the recurrent mixers (blocks of 64 tokens on the matrix instruction), decode-sized steps the token-by-token form
    const bool lin_chunked = max_count >= 32;
    for (const SvLayer& l : s->L) {
        const kr_serve_layer& d = l.d;
        if (d.proj_conv) max_pconv = std::max(max_pconv, (size_t)l.pconv_c());
        if (l.has_ssd()) {
            max_sconv = std::max(max_sconv, (size_t)l.ssd_conv_c()); max_lin = std::max(max_lin, (size_t)l.ssd_inner());
            if (lin_chunked && kr_sv_lin_chunked_fits(d.ssd_state, d.ssd_vdim)) {
                lin_tok = std::max(lin_tok, (size_t)d.ssd_heads); lin_sb = std::max(lin_sb, (size_t)d.ssd_heads * d.ssd_state * d.ssd_vdim); lin_nb = std::max(lin_nb, (size_t)d.ssd_heads * d.ssd_state);
                max_ssdz = std::max(max_ssdz, (size_t)d.ssd_heads * (2 * d.ssd_state + d.ssd_vdim));
            }
        }
        if (l.gla()) { max_ga1 = std::max(max_ga1, (size_t)d.decay_rank); max_gz = std::max(max_gz, (size_t)d.heads * d.dim); }
        if (l.recurrent()) {
            max_lin = std::max(max_lin, (size_t)d.heads * d.vdim);
            if (lin_chunked && l.chunkable() && kr_sv_lin_chunked_fits(d.dim, d.vdim)) {
                lin_tok = std::max(lin_tok, (size_t)d.heads); lin_sb = std::max(lin_sb, (size_t)d.heads * d.dim * d.vdim); lin_nb = std::max(lin_nb, (size_t)d.heads * d.dim);
            }
        }
        if (d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE) whole_norm = true;
        max_qkv = std::max(max_qkv, (size_t)l.n_h); max_att = std::max(max_att, std::max((size_t)d.heads * l.att_vdim(), (size_t)l.o_cols()));
        if (d.v_mix) max_vf = std::max(max_vf, (size_t)d.kv_heads * d.vdim);
        if (l.latent()) {
            lq_c = std::max(lq_c, (size_t)d.q_rank); lq_2 = std::max(lq_2, (size_t)d.heads * (d.dim + d.rot_dims)); lq_n = std::max(lq_n, (size_t)d.heads * d.dim);
            lq_e = std::max(lq_e, (size_t)d.heads * l.att_dim()); att2 = std::max(att2, (size_t)d.heads * d.vdim); head_i = std::max(head_i, (size_t)d.heads);
        }
        if (d.mlp_kind == KR_SERVE_MLP_DENSE) { max_gu = std::max(max_gu, (size_t)2 * d.ff); max_y = std::max(max_y, (size_t)d.ff); }
        if (d.mlp_kind == KR_SERVE_MLP_MOE) {
            max_gu = std::max(max_gu, std::max((size_t)d.top * 2 * d.expert_ff, (size_t)2 * d.shared_ff));
            max_y = std::max(max_y, std::max((size_t)d.top * d.expert_ff, (size_t)d.shared_ff));
            max_rows = std::max(max_rows, (size_t)d.top * W); max_pairs = std::max(max_pairs, (size_t)d.top); max_E = std::max(max_E, d.experts);
        }
    }
    const size_t Ts = (size_t)T;
    if (s->x.ensure(Ts * W * 4) || s->h.ensure(Ts * W * s->esz) || s->qkv.ensure(Ts * max_qkv * 4) || s->att.ensure(Ts * max_att * s->esz) || s->mix.ensure(Ts * W * 4) ||
        s->gu.ensure(Ts * max_gu * 4 + 16) || s->y.ensure(Ts * max_y * s->esz + 16) || s->rows.ensure(Ts * max_rows * 4 + 16) || s->ffout.ensure(Ts * W * 4) ||
        s->ids.ensure(Ts * max_pairs * 4 + 16) || s->rz.ensure(Ts * (size_t)max_E * 8 + 16) || s->wts.ensure(Ts * max_pairs * 4 + 16) || s->moe_i.ensure((Ts * max_pairs * 3 + 3 * (size_t)max_E + 8) * 4) ||
        s->hw.ensure((size_t)std::max(n_want, 1) * W * s->esz) || s->logits.ensure((size_t)std::max(n_want, 1) * c.vocab * 4) || s->amax.ensure((size_t)std::max(n_want, 1) * 4))
        return kr_fail(KR_ERR_HIP, "step scratch for %d tokens", T);
    if ((max_vf && s->v_first.ensure(Ts * max_vf * 4)) ||
        (head_i && (s->lq_c.ensure(Ts * lq_c * s->esz) || s->lq_2.ensure(Ts * lq_2 * 4) || s->lq_n.ensure(Ts * lq_n * s->esz) || s->lq_e.ensure(Ts * lq_e * 4) ||
                    s->att2.ensure(Ts * att2 * s->esz) || s->head_i.ensure((2 * Ts * head_i + head_i + 1) * 4))))
        return kr_fail(KR_ERR_HIP, "mixer scratch for %d tokens", T);
    if ((c.canon_taps > 1 && (s->h32.ensure(Ts * W * 4) || s->hc.ensure(Ts * W * s->esz))) || (c.res_gate && s->rg.ensure(Ts * W * 4)) || (whole_norm && s->qk_rms.ensure(Ts * 2 * 4)) ||
        (max_lin && s->lin_o.ensure(Ts * max_lin * 4)) ||
        (lin_tok && (s->lin_tok.ensure(Ts * lin_tok * 16) || s->lin_sbuf.ensure((size_t)n_chunks * lin_sb * 4) || s->lin_nbuf.ensure((size_t)n_chunks * lin_nb * 4) || s->lin_cm.ensure((size_t)n_chunks * lin_tok * 16))))
        return kr_fail(KR_ERR_HIP, "block scratch for %d tokens", T);
    if ((max_pconv && s->qkv2.ensure(Ts * max_pconv * 4)) || (max_sconv && s->sconv.ensure(Ts * max_sconv * 4)) || (max_ga1 && (s->ga1.ensure(Ts * max_ga1 * s->esz) || s->gz.ensure(Ts * max_gz * 4))))
        return kr_fail(KR_ERR_HIP, "convolution / decay scratch for %d tokens", T);
    if (max_ssdz && s->ssd_z.ensure(Ts * max_ssdz * 4)) return kr_fail(KR_ERR_HIP, "state-space block scratch for %d tokens", T);
    for (SvRope& r : s->ropes) if (r.cs.ensure(Ts * (r.dims / 2) * 8)) return kr_fail(KR_ERR_HIP, "rope table");
    if (s->capture) { if (s->cap.ensure((size_t)c.n_layers * Ts * W * 4)) return kr_fail(KR_ERR_HIP, "capture buffer"); s->cap_T = T; }
    std::vector<int> nsplit(c.n_layers, 1);
    for (int li = 0; li < c.n_layers; li++) {
        const SvLayer& l = s->L[li]; const kr_serve_layer& d = l.d;
        if (l.recurrent() || l.ssd_alone()) continue;
        const int visible = d.window > 0 ? std::min(max_pos + 1, d.window) : (d.chunk > 0 ? std::min(max_pos + 1, d.chunk) : max_pos + 1);
        const int ldk = l.latent() ? l.att_dim() : d.kv_heads * d.dim, ldv = l.latent() ? l.att_dim() : d.kv_heads * d.vdim;
        nsplit[li] = kr_sv_attention_splits(T, d.heads, l.att_heads_kv(), l.att_dim(), l.att_vdim(), ldk, ldv, s->f32, visible);
        if (nsplit[li] > 1 && (s->part_ml.ensure(Ts * d.heads * nsplit[li] * 8) || s->part_acc.ensure(Ts * d.heads * nsplit[li] * l.att_vdim() * 4)))
            return kr_fail(KR_ERR_HIP, "attention split scratch");
    }
    const bool want_amax = argmax_out != nullptr;
    // every launch of the step, in order; no allocation, no host copy: the same body runs eagerly or under stream capture
    auto enqueue = [&]() -> int {
    float* x = (float*)s->x.p;
    {
        Timer tm(s, 7);
        kr_sv_embed(s->embed.p, s->f32, d_tok, x, c.pre_norm ? nullptr : s->h.p, T, W, c.embed_scale != 0.0f ? c.embed_scale : 1.0f, c.bigram_buckets > 0 ? s->bigram.p : nullptr, d_brow,
                    st);     // without input norms the first sublayer reads the embedding row itself
    }
    if (c.embed_norm) { Timer tm(s, 0); kr_sv_stream_norm(x, nullptr, (const float*)s->enorm_w.p, nullptr, true, nullptr, s->f32, T, W, c.norm_eps, c.norm_kind, c.norm_groups > 1 ? c.norm_groups : 1, st); }
    {
        Timer tm(s, 2);
        for (SvRope& r : s->ropes) kr_sv_rope_table(d_pos, (const double*)r.inv_freq.p, (float2*)r.cs.p, T, r.dims / 2, r.mult, st);
    }
    int* mi = (int*)s->moe_i.p;
    // down projection of a gated feed-forward: decode-sized problems form the activation inside the projection's launch, larger ones write it once
    auto down_proj = [&](KrSvGemm g, const float* gu, int ld, int rows_m, int F, int kind, float limit, float alpha) {
        if (kr_sv_gemm_small(g)) { g.act_gu = gu; g.act_ld = ld; g.act_kind = kind; g.act_limit = limit; g.act_alpha = alpha; g.A = nullptr; Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); return; }
        { Timer tm(s, 5); kr_sv_act(gu, ld, s->y.p, s->f32, rows_m, F, kind, limit, alpha, st); }
        g.A = s->y.p; g.lda = F;
        { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
    };
    // the residual sum that ends a sublayer (or, in a parallel block, the layer); `next`: the norm of the sublayer that reads the new x, null with
    // hand_on = the row as it is, or nothing when no sublayer follows
    const int NG = c.norm_groups > 1 ? c.norm_groups : 1;
    const bool canon = c.canon_taps > 1;
    // gate: 0 none, 1 the mixer's (logits in rg, the output projection's bias, and the input convolution's rows of this layer are kept), 2 the feed-forward's
    // (logits in the last row block of hz).  to_mixer: the handed-on row feeds a mixer (an f32 copy goes along for its input convolution)
    const SvLayer* res_layer = nullptr; const SvLayer* res_run = nullptr; int res_gate_kind = 0; bool res_to_mixer = false;
    auto residual = [&](const float* mixp, const float* dense, const float* shared, const float* rows, const int* pair_pos, int top, const DevBuf* post_w, const DevBuf* post_b,
                        bool hand_on, const DevBuf* next_w, const DevBuf* next_b) {
        Timer tm(s, 6);
        KrSvResidual r{};
        r.groups = NG;
        if (res_layer) {
            const SvLayer& rl = *res_layer;
            if (mixp && rl.d.proj_bias) r.mix_bias = (const float*)rl.o_bias.p;
            if (res_gate_kind == 1) {
                if (c.res_gate) { r.gate = (const float*)s->rg.p; r.ld_gate = W; r.gate_b = (const float*)rl.rg1_b.p; }
                if (canon) { r.h32_in = (const float*)s->h32.p; r.canon_state = (float*)res_run->canon_state.p; r.canon_keep = c.canon_taps - 1; r.slot = d_slot; r.pos = d_pos; }
            } else if (res_gate_kind == 2 && c.res_gate) { r.gate = (const float*)s->qkv.p + rl.off_rg2; r.ld_gate = rl.n_h; r.gate_b = (const float*)rl.rg2_b.p; }
        }
        if (canon && hand_on && res_to_mixer) r.h32_out = (float*)s->h32.p;
        r.x = x; r.mix = mixp; r.dense = dense; r.shared = shared; r.rows = rows; r.pair_pos = pair_pos; r.wts = (const float*)s->wts.p; r.top = top;
        r.post_w = post_w ? (const float*)post_w->p : nullptr; r.post_b = (post_w && c.norm_bias && post_b) ? (const float*)post_b->p : nullptr; r.mult = c.residual_mult;
        r.norm_w = (hand_on && next_w) ? (const float*)next_w->p : nullptr; r.norm_b = (hand_on && next_w && c.norm_bias && next_b) ? (const float*)next_b->p : nullptr;
        r.h_out = hand_on ? s->h.p : nullptr; r.T = T; r.width = W; r.kind = c.norm_kind; r.eps = c.norm_eps;
        kr_sv_residual_norm(r, s->f32, st);
    };
    if (c.pre_norm && !s->L[0].d.pre_add) {
        Timer tm(s, 0);
        kr_sv_norm(x, nullptr, (const float*)s->L[0].norm_w.p, c.norm_bias ? (const float*)s->L[0].norm_b.p : nullptr, s->h.p, s->f32, T, W, c.norm_eps, c.norm_kind, NG,
                   canon ? (float*)s->h32.p : nullptr, st);
    }
    int head_rows_for = 0;               // the head row tables in head_i are valid for this head count
    for (int li = 0; li < c.n_layers; li++) {
        SvLayer& run = s->L[li];                         // cache pools, state and the vector before the layer: this run's own
        SvLayer& l = s->L[run.wsrc]; const kr_serve_layer& d = l.d;       // tensors and layout: the layer that owns them
        const SvLayer* nxrun = li + 1 < c.n_layers ? &s->L[li + 1] : nullptr;
        const SvLayer* nx = nxrun ? &s->L[nxrun->wsrc] : nullptr;
        const bool hand = nxrun && !nxrun->d.pre_add;     // a layer with a vector before it forms its own input from the stream
        const bool has_ff = d.mlp_kind != KR_SERVE_MLP_NONE;
        if (run.d.pre_add) {
            Timer tm(s, 0);
            kr_sv_stream_norm(x, (const float*)run.pre_add.p, (const float*)l.norm_w.p, c.norm_bias ? (const float*)l.norm_b.p : nullptr, false, s->h.p, s->f32, T, W, c.norm_eps, c.norm_kind, NG, st);
        }
        float* hz = (float*)s->qkv.p;                    // [T, n_h]: q | k | v (or the latents) | router logits | gate | up of this layer
        KrSvGemm g{};
        // a parallel block multiplies its one input by every matrix at once; a sequential block's feed-forward reads the x its mixer leaves
        const void* mixer_in = s->h.p;
        if (canon) {       // the mixer reads h + conv(h); the residual gate below reads h itself
            KrSvCanon cv{}; cv.h32 = (const float*)s->h32.p; cv.w = (const float*)l.canon.p; cv.taps = c.canon_taps; cv.state = (float*)run.canon_state.p;
            cv.slot = d_slot; cv.pos = d_pos; cv.T = T; cv.width = W; cv.out = s->hc.p;
            Timer tm(s, 0); kr_sv_canon(cv, s->f32, st);
            mixer_in = s->hc.p;
        }
        if (c.res_gate) {
            KrSvGemm gg{}; gg.A = s->h.p; gg.lda = W; gg.W = l.rg1.p; gg.C = (float*)s->rg.p; gg.ldc = W; gg.M = T; gg.N = W; gg.K = W;
            Timer tm(s, 1); kr_sv_gemm(gg, s->f32, st);
        }
        g.A = mixer_in; g.lda = W; g.W = l.hw.p; g.C = hz; g.ldc = l.n_h; g.M = T; g.N = seq ? l.n_qkv : l.n_h; g.K = W;
        { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
        const SvLayer& kvl = d.kv_from >= 0 ? s->L[d.kv_from] : run;
        KrSvAttn a{};
        a.heads = d.heads; a.kv_heads = l.att_heads_kv(); a.dim = l.att_dim(); a.vdim = l.att_vdim();
        a.eps = c.norm_eps; a.scale = d.scale; a.window = d.window; a.chunk = d.chunk; a.slopes = d.dist_bias ? (const float*)l.slopes.p : nullptr;
        a.sink = d.has_sink ? (const float*)l.sink.p : nullptr;
        a.kpool = kvl.kpool.p; a.page_table = d_tab; a.table_ld = s->n_pages; a.slot = d_slot; a.pos = d_pos; a.page_tokens = PT; a.T = T;
        a.out = s->att.p;
        a.nsplit = nsplit[li]; a.part_ml = (float*)s->part_ml.p; a.part_acc = (float*)s->part_acc.p;
        const void* o_in = s->att.p;
        if (l.recurrent()) {
            KrSvLin q{};
            q.kind = d.mixer_kind; q.z = hz; q.ld = l.n_h; q.heads = d.heads; q.dim = d.dim; q.vdim = d.vdim; q.rot_dims = d.rot_dims;
            q.cs = d.rot_dims ? (const float2*)s->ropes[l.rope_id].cs.p : nullptr;
            const float isd = (float)(1.0 / std::sqrt((double)d.dim));
            q.q_scale = d.mixer_kind == KR_SERVE_MIX_MLSTM ? isd : 1.0f; q.k_scale = d.mixer_kind == KR_SERVE_MIX_RETENTION ? isd : 1.0f;
            q.decay = (const float*)l.decay.p; q.i_bias = (const float*)l.i_bias.p; q.f_bias = (const float*)l.f_bias.p; q.gate_cap = d.gate_cap;
            q.state = (float*)run.lin_state.p; q.state_stride = l.lin_state_stride; q.nm = (float*)run.lin_nm.p; q.nm_stride = l.lin_nm_stride;
            q.ent_off = d_eoff; q.ent_slot = d_eslot; q.n_entries = n_entries; q.pos = d_pos; q.T = T;
            q.o = (float*)s->lin_o.p; q.norm_w = d.lin_norm_weight ? (const float*)l.lin_norm.p : nullptr; q.norm_shared = d.lin_norm_weight == 2; q.eps = c.norm_eps; q.out = s->att.p;
            if (l.gla()) {
                // the decays' logits: a low-rank pair of projections, the first one's output in the storage type; q scaled, the decay itself formed in the scan
                KrSvGemm g1{}; g1.A = mixer_in; g1.lda = W; g1.W = l.a1.p; g1.C = (float*)s->ga1.p; g1.ldc = d.decay_rank; g1.c_storage = 1; g1.M = T; g1.N = d.decay_rank; g1.K = W;
                KrSvGemm g2{}; g2.A = s->ga1.p; g2.lda = d.decay_rank; g2.W = l.a2.p; g2.C = (float*)s->gz.p; g2.ldc = d.heads * d.dim; g2.M = T; g2.N = g2.ldc; g2.K = d.decay_rank;
                { Timer tm(s, 1); kr_sv_gemm(g1, s->f32, st); kr_sv_gemm(g2, s->f32, st); }
                q.qsrc = hz; q.ksrc = hz + (size_t)d.heads * d.dim; q.vsrc = hz + (size_t)2 * d.heads * d.dim; q.src_ld = l.n_h; q.qk_group = 1;
                q.gz = (const float*)s->gz.p; q.gz_ld = d.heads * d.dim; q.gz_bias = (const float*)l.a2_b.p; q.inv_tau = 1.0f / d.decay_tau;
                q.q_scale = isd; q.k_scale = 1.0f;
            }
            q.ent_chunk0 = d_echunk; q.n_chunks = n_chunks; q.tok = (float4*)s->lin_tok.p; q.sbuf = (float*)s->lin_sbuf.p; q.nbuf = (float*)s->lin_nbuf.p; q.cmeta = (float*)s->lin_cm.p;
            {
                Timer tm(s, 3);
                if (lin_chunked && l.chunkable() && kr_sv_lin_chunked_fits(d.dim, d.vdim)) kr_sv_lin_chunked(q, st);
                else if (lin_chunked && kr_sv_lin_scan_wide_fits(q.kind, d.dim)) kr_sv_lin_scan_wide(q, st);
                else kr_sv_lin_scan(q, st);
            }
            { Timer tm(s, 2); kr_sv_lin_out(q, s->f32, st); }
        } else if (l.ssd_alone()) {
            // no first mixer: the state-space mixer below is the layer's only one
        } else if (!l.latent()) {
            a.qkv = hz; a.ldq = l.n_h; a.rot_dims = d.rot_dims; a.rot_interleaved = d.rot_interleaved; a.unit_norm = d.qk_unit_norm; a.own_kv = d.kv_from < 0;
            a.q_norm_w = (const float*)l.q_norm.p; a.k_norm_w = (const float*)l.k_norm.p;
            a.cs = d.rot_dims ? (const float2*)s->ropes[l.rope_id].cs.p : nullptr;
            a.vpool = kvl.vpool.p; a.ldk = d.kv_heads * d.dim; a.ldv = d.kv_heads * d.vdim;
            a.v_mix = d.v_mix; a.v_lambda = (const float*)l.vmix.p; a.v_first = (float*)s->v_first.p;
            a.q_bias = d.proj_bias ? (const float*)l.q_bias.p : nullptr; a.k_bias = (d.proj_bias && d.kv_from < 0) ? (const float*)l.k_bias.p : nullptr;
            a.inv_rms = a.inv_rms_out = (float*)s->qk_rms.p; a.v_from_k = d.v_from_k; a.softcap = d.softcap;
            if (d.out_gate) { a.out_gate = hz + l.off_ogate; a.ld_gate = l.n_h; a.gate_elem = d.out_gate == KR_SERVE_OGATE_ELEM_SIGMOID; }
            a.v_bias = d.proj_bias == 2 ? (const float*)l.v_bias.p : nullptr;
            if (l.has_ssd()) { a.out_ld = l.o_cols(); a.out_scale = d.mix_scale; }
            if (d.proj_conv) {
                // q | k | v with their biases pass the short convolution; the preparation below reads the convolved rows and adds no bias again
                KrSvChanConv cv{}; cv.in = hz; cv.ld_in = l.n_h; cv.in_bias = d.proj_bias ? (const float*)l.pconv_bias.p : nullptr; cv.w = (const float*)l.pconv_w.p; cv.taps = d.proj_conv;
                cv.out = (float*)s->qkv2.p; cv.ld_out = l.pconv_c(); cv.state = (float*)run.pconv_state.p; cv.slot = d_slot; cv.pos = d_pos; cv.T = T; cv.C = l.pconv_c();
                cv.ent_off = d_eoff; cv.n_entries = n_entries;
                Timer tm(s, 2); kr_sv_chan_conv(cv, st); kr_sv_chan_conv_save(cv, st);
                a.qkv = (float*)s->qkv2.p; a.ldq = l.pconv_c(); a.q_bias = a.k_bias = a.v_bias = nullptr;
            }
            if (d.qk_unit_norm == KR_SERVE_QKNORM_WHOLE) { Timer tm(s, 2); kr_sv_qk_rms(a, st); }
            { Timer tm(s, 2); kr_sv_qk_prep(a, s->f32, st); }
            { Timer tm(s, 3); kr_sv_attention(a, s->f32, st); }
        } else {
            // queries: norm the latent, W_uq, turn the rotated part, fold W_uk of every head into the plain part; keys / values: the normed latent and the
            // turned shared part are the cache row, read by the attention kernels as ONE key / value head whose values are the leading kv_rank of the key row
            const int H = d.heads, R = d.kv_rank, De = l.att_dim();
            KrSvLatent q{};
            q.dz = hz; q.ld = l.n_h; q.q_rank = d.q_rank; q.kv_rank = R; q.rot = d.rot_dims; q.heads = H; q.dim = d.dim;
            q.dq_norm_w = (const float*)l.dq_norm.p; q.dkv_norm_w = (const float*)l.dkv_norm.p; q.eps = c.norm_eps;
            q.cs = d.rot_dims ? (const float2*)s->ropes[l.rope_id].cs.p : nullptr; q.cq = s->lq_c.p;
            q.pool = l.kpool.p; q.page_table = d_tab; q.table_ld = s->n_pages; q.slot = d_slot; q.pos = d_pos; q.page_tokens = PT; q.T = T;
            int* hseg = (int*)s->head_i.p; int* hrows = hseg + H + 1; int* hgroup = hrows + (size_t)T * H;
            {
                Timer tm(s, 2);
                kr_sv_latent_prep(q, s->f32, st);
                if (head_rows_for != H) { kr_sv_head_rows(T, H, hseg, hrows, hgroup, st); head_rows_for = H; }
            }
            g = KrSvGemm{}; g.A = s->lq_c.p; g.lda = d.q_rank; g.W = l.uq.p; g.C = (float*)s->lq_2.p; g.ldc = H * (d.dim + d.rot_dims); g.M = T; g.N = g.ldc; g.K = d.q_rank;
            { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
            { Timer tm(s, 2); kr_sv_latent_q(q, (const float*)s->lq_2.p, s->lq_n.p, (float*)s->lq_e.p, s->f32, st); }
            g = KrSvGemm{}; g.A = s->lq_n.p; g.lda = d.dim; g.a_rows = hrows; g.W = l.ukT.p; g.w_stride = (size_t)R * d.dim; g.C = (float*)s->lq_e.p; g.ldc = De; g.c_rows = hrows;
            g.M = T * H; g.N = R; g.K = d.dim; g.seg = hseg; g.row_group = hgroup; g.n_groups = H; g.rowwise_upto = 16 * H;
            { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
            a.qkv = (float*)s->lq_e.p; a.ldq = H * De; a.vpool = l.kpool.p; a.ldk = De; a.ldv = De;
            { Timer tm(s, 3); kr_sv_attention(a, s->f32, st); }
            g = KrSvGemm{}; g.A = s->att.p; g.lda = R; g.a_rows = hrows; g.W = l.uv.p; g.w_stride = (size_t)d.vdim * R; g.C = (float*)s->att2.p; g.ldc = d.vdim; g.c_rows = hrows; g.c_storage = 1;
            g.M = T * H; g.N = d.vdim; g.K = R; g.seg = hseg; g.row_group = hgroup; g.n_groups = H; g.rowwise_upto = 16 * H;
            { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
            o_in = s->att2.p;
        }
        if (l.has_ssd()) {
            // [z | x | B | C | dt] came out of the layer's one GEMM; x | B | C pass their convolution, the scan keeps S [state, vdim] per head in registers, and the
            // gated, normed output lands beside the first mixer's so that ONE output projection over [first | state-space] forms the layer's mixer output
            const int inner = l.ssd_inner(), gn = d.ssd_groups * d.ssd_state, cc = l.ssd_conv_c();
            float* zin = hz + l.off_ssd;
            KrSvChanConv cv{}; cv.in = zin + inner; cv.ld_in = l.n_h; cv.w = (const float*)l.sconv_w.p; cv.taps = d.ssd_conv; cv.cb = (const float*)l.sconv_b.p; cv.act = 1;
            cv.out = (float*)s->sconv.p; cv.ld_out = cc; cv.state = (float*)run.sconv_state.p; cv.slot = d_slot; cv.pos = d_pos; cv.T = T; cv.C = cc; cv.ent_off = d_eoff; cv.n_entries = n_entries;
            { Timer tm(s, 2); kr_sv_chan_conv(cv, st); kr_sv_chan_conv_save(cv, st); }
            KrSvLin q{};
            q.kind = KR_SERVE_MIX_SSD; q.heads = d.ssd_heads; q.dim = d.ssd_state; q.vdim = d.ssd_vdim; q.q_scale = q.k_scale = 1.0f;
            q.vsrc = (const float*)s->sconv.p; q.ksrc = q.vsrc + inner; q.qsrc = q.ksrc + gn; q.src_ld = cc; q.qk_group = d.ssd_heads / d.ssd_groups;
            q.dtz = zin + inner + cc; q.dtz_ld = l.n_h; q.dt_bias = (const float*)l.dt_bias.p; q.a_log = (const float*)l.a_log.p;
            q.state = (float*)run.ssd_state.p; q.state_stride = l.ssd_state_stride;
            q.ent_off = d_eoff; q.ent_slot = d_eslot; q.n_entries = n_entries; q.pos = d_pos; q.T = T; q.o = (float*)s->lin_o.p;
            {
                Timer tm(s, 3);
                if (lin_chunked && kr_sv_lin_chunked_fits(d.ssd_state, d.ssd_vdim)) {
                    // prompt portions: a retention with a decay per token, on the block launches of the recurrent mixers (same state layout)
                    const int ldz = d.ssd_heads * (2 * d.ssd_state + d.ssd_vdim);
                    q.tok = (float4*)s->lin_tok.p;
                    kr_sv_ssd_expand(q, (float*)s->ssd_z.p, ldz, st);
                    KrSvLin c2{};
                    c2.kind = KR_SERVE_MIX_RETENTION; c2.prepped = 1; c2.z = (float*)s->ssd_z.p; c2.ld = ldz; c2.heads = d.ssd_heads; c2.dim = d.ssd_state; c2.vdim = d.ssd_vdim;
                    c2.q_scale = c2.k_scale = 1.0f; c2.state = q.state; c2.state_stride = q.state_stride; c2.ent_off = d_eoff; c2.ent_slot = d_eslot; c2.n_entries = n_entries;
                    c2.pos = d_pos; c2.T = T; c2.o = q.o; c2.ent_chunk0 = d_echunk; c2.n_chunks = n_chunks; c2.tok = q.tok; c2.sbuf = (float*)s->lin_sbuf.p;
                    c2.nbuf = (float*)s->lin_nbuf.p; c2.cmeta = (float*)s->lin_cm.p;
                    kr_sv_lin_chunked(c2, st);
                } else if (lin_chunked && kr_sv_lin_scan_wide_fits(q.kind, q.dim)) kr_sv_lin_scan_wide(q, st);
                else kr_sv_lin_scan(q, st);
            }
            KrSvSsdOut so{};
            so.o = (const float*)s->lin_o.p; so.x = (const float*)s->sconv.p; so.ld_x = cc; so.z = zin; so.ld_z = l.n_h; so.D = (const float*)l.ssd_d.p; so.w = (const float*)l.ssd_norm.p;
            so.heads = d.ssd_heads; so.vdim = d.ssd_vdim; so.groups = d.ssd_norm_groups; so.eps = c.norm_eps;
            so.scale = (d.side_mixer && d.side_scale != 0.0f) ? d.side_scale : 1.0f;
            so.out = (char*)s->att.p + (size_t)l.att_out_cols() * s->esz; so.out_ld = l.o_cols(); so.T = T;
            { Timer tm(s, 2); kr_sv_ssd_out(so, s->f32, st); }
        }
        g = KrSvGemm{};
        g.A = o_in; g.lda = l.latent() ? d.heads * d.vdim : l.o_cols(); g.W = l.o.p; g.C = (float*)s->mix.p; g.ldc = W; g.M = T; g.N = W; g.K = g.lda;
        { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
        if (seq) {
            // the mixer's sublayer ends here; the new x, normed or as it is, is the feed-forward's input (or the next layer's when there is none)
            res_layer = &l; res_run = &run; res_gate_kind = 1; res_to_mixer = !has_ff;
            if (has_ff) residual((const float*)s->mix.p, nullptr, nullptr, nullptr, nullptr, 0, c.post_norm ? &l.post1_w : nullptr, &l.post1_b, true, c.pre_norm ? &l.norm2_w : nullptr, &l.norm2_b);
            else residual((const float*)s->mix.p, nullptr, nullptr, nullptr, nullptr, 0, c.post_norm ? &l.post1_w : nullptr, &l.post1_b, hand, (nx && c.pre_norm) ? &nx->norm_w : nullptr,
                          nx ? &nx->norm_b : nullptr);
            if (has_ff && l.n_h > l.off_router) {
                g = KrSvGemm{}; g.A = s->h.p; g.lda = W; g.W = (const char*)l.hw.p + (size_t)l.off_router * W * s->esz; g.C = hz + l.off_router; g.ldc = l.n_h; g.M = T; g.N = l.n_h - l.off_router; g.K = W;
                Timer tm(s, 1); kr_sv_gemm(g, s->f32, st);
            }
        }
        const float *dense = nullptr, *shared = nullptr, *rows = nullptr; const int* pair_pos = nullptr;
        if (d.mlp_kind == KR_SERVE_MLP_DENSE) {
            g = KrSvGemm{}; g.W = l.down.p; g.C = (float*)s->ffout.p; g.ldc = W; g.M = T; g.N = W; g.K = d.ff;
            down_proj(g, hz + l.off_gu, l.n_h, T, d.ff, d.dense_act, 0.0f, 1.0f);
            dense = (const float*)s->ffout.p;
        } else if (d.mlp_kind == KR_SERVE_MLP_MOE) {
            const int E = d.experts, top = d.top, F = d.expert_ff, P = T * top;
            int* counts_d = mi; int* seg = mi + E; int* cursor = seg + E + 1; int* src_row = cursor + E; int* row_group = src_row + P; int* pp = row_group + P;
            {
                Timer tm(s, 4);
                kr_sv_router_select(hz + l.off_router, l.n_h, s->f32 ? 1 : 2, d.router_bias ? (const float*)l.router_b.p : nullptr, d.router_bias, d.router_score, d.group_score, T, E, top,
                                    d.groups, d.keep, d.renorm, (int*)s->ids.p, (float*)s->wts.p, st);
                kr_sv_moe_sort((const int*)s->ids.p, T, top, E, counts_d, seg, cursor, src_row, row_group, pp, st);
            }
            g = KrSvGemm{}; g.A = s->h.p; g.lda = W; g.W = l.egu.p; g.w_stride = (size_t)2 * F * W; g.C = (float*)s->gu.p; g.ldc = 2 * F; g.M = P; g.N = 2 * F; g.K = W;
            g.a_rows = src_row; g.seg = seg; g.row_group = row_group; g.n_groups = E;
            { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
            g = KrSvGemm{}; g.W = l.edown.p; g.w_stride = (size_t)W * F; g.C = (float*)s->rows.p; g.ldc = W; g.M = P; g.N = W; g.K = F;
            g.seg = seg; g.row_group = row_group; g.n_groups = E;
            down_proj(g, (const float*)s->gu.p, 2 * F, P, F, d.expert_act, d.expert_limit, d.expert_alpha);
            rows = (const float*)s->rows.p; pair_pos = pp;
            if (d.shared_ff > 0) {
                const int SF = d.shared_ff;
                g = KrSvGemm{}; g.W = l.sdown.p; g.C = (float*)s->ffout.p; g.ldc = W; g.M = T; g.N = W; g.K = SF;
                down_proj(g, hz + l.off_gu, l.n_h, T, SF, d.expert_act, d.shared_limit, d.expert_alpha);
                shared = (const float*)s->ffout.p;
            }
        }
        // x += the layer's sublayers (parallel block) or the feed-forward alone (sequential), and the next layer's input from the same launch
        res_layer = &l; res_run = &run; res_gate_kind = seq ? 2 : 0; res_to_mixer = true;
        if (!seq) residual((const float*)s->mix.p, dense, shared, rows, pair_pos, d.top, nullptr, nullptr, hand, (nx && c.pre_norm) ? &nx->norm_w : nullptr, nx ? &nx->norm_b : nullptr);
        else if (has_ff) residual(nullptr, dense, shared, rows, pair_pos, d.top, c.post_norm ? &l.post2_w : nullptr, &l.post2_b, hand, (nx && c.pre_norm) ? &nx->norm_w : nullptr,
                                  nx ? &nx->norm_b : nullptr);
        if (s->capture) KR_HIP(hipMemcpyAsync((float*)s->cap.p + (size_t)li * Ts * W, x, Ts * W * 4, hipMemcpyDeviceToDevice, st));
    }
    if (n_want > 0) {
        { Timer tm(s, 0); kr_sv_norm(x, d_want, (const float*)s->fnorm_w.p, c.norm_bias ? (const float*)s->fnorm_b.p : nullptr, s->hw.p, s->f32, n_want, W, c.norm_eps, c.norm_kind, NG, nullptr, st); }
        KrSvGemm g{}; g.A = s->hw.p; g.lda = W; g.W = s->head.p; g.C = (float*)s->logits.p; g.ldc = c.vocab; g.M = n_want; g.N = c.vocab; g.K = W;
        { Timer tm(s, 1); kr_sv_gemm(g, s->f32, st); }
        if (c.logit_scale != 0.0f && c.logit_scale != 1.0f) { Timer tm(s, 7); kr_sv_scale((float*)s->logits.p, (size_t)n_want * c.vocab, c.logit_scale, st); }
        if (want_amax) { Timer tm(s, 7); kr_sv_argmax((const float*)s->logits.p, n_want, c.vocab, (int*)s->amax.p, st); }
    }
    return KR_OK;
    };   // enqueue
    bool decode_shaped = s->use_graph && !s->prof && !s->capture && T <= 64;
    for (int e = 0; e < n_entries && decode_shaped; e++) decode_shaped = counts[e] == 1;
    bool done = false;
    if (decode_shaped) {
        // the key: everything a launch argument depends on -- batch, wanted rows, the split of every layer, the scratch addresses
        uint64_t key = 1469598103934665603ull;
        auto mixin = [&](uint64_t v) { key = (key ^ v) * 1099511628211ull; };
        mixin((uint64_t)T); mixin((uint64_t)n_want); mixin(want_amax);
        for (int v : nsplit) mixin((uint64_t)v);
        for (const DevBuf* b : {&s->meta, &s->x, &s->h, &s->qkv, &s->att, &s->mix, &s->gu, &s->y, &s->rows, &s->ffout, &s->ids, &s->wts, &s->rz, &s->moe_i, &s->hw, &s->logits,
                                &s->amax, &s->part_ml, &s->part_acc, &s->v_first, &s->lq_c, &s->lq_2, &s->lq_n, &s->lq_e, &s->att2, &s->head_i, &s->h32, &s->hc, &s->rg, &s->qk_rms, &s->lin_o, &s->qkv2, &s->sconv, &s->ga1, &s->gz}) mixin((uint64_t)(uintptr_t)b->p);
        for (const SvRope& r : s->ropes) mixin((uint64_t)(uintptr_t)r.cs.p);
        hipGraphExec_t exec = nullptr;
        for (auto& g : s->graphs) if (g.key == key) exec = g.exec;
        if (!exec) {
            int visits = 0;
            for (auto& q : s->seen) if (q.first == key) visits = ++q.second;
            if (!visits) { if (s->seen.size() > 4096) s->seen.clear(); s->seen.emplace_back(key, 1); }
            if (visits >= 2) {
                if (s->graphs.size() >= 64) { for (auto& g : s->graphs) (void)hipGraphExecDestroy(g.exec); s->graphs.clear(); }
                hipGraph_t graph = nullptr;
                KR_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
                const int rc = enqueue();
                const hipError_t ee = hipStreamEndCapture(st, &graph);
                if (rc) { if (graph) (void)hipGraphDestroy(graph); return rc; }
                if (ee != hipSuccess) return kr_fail(KR_ERR_HIP, "hipStreamEndCapture failed: %s", hipGetErrorString(ee));
                const hipError_t ie = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
                (void)hipGraphDestroy(graph);
                if (ie != hipSuccess) return kr_fail(KR_ERR_HIP, "hipGraphInstantiate failed: %s", hipGetErrorString(ie));
                s->graphs.push_back({key, exec});
            }
        }
        if (exec) { KR_HIP(hipGraphLaunch(exec, st)); s->graph_replays++; done = true; }
    }
    if (!done) { const int rc = enqueue(); if (rc) return rc; }
    if (n_want > 0) {
        if (logits_out) KR_HIP(hipMemcpyAsync(logits_out, s->logits.p, (size_t)n_want * c.vocab * 4, hipMemcpyDeviceToHost, st));
        if (argmax_out) KR_HIP(hipMemcpyAsync(argmax_out, s->amax.p, (size_t)n_want * 4, hipMemcpyDeviceToHost, st));
    }
    s->last_want = n_want;
    KR_HIP(hipStreamSynchronize(st));
    KR_HIP(hipGetLastError());
    return KR_OK;
}

int kr_serve_set_use_graph(kr_serve* s, int enable) { if (!s) return kr_fail(KR_ERR_VALUE, "null argument"); s->use_graph = enable != 0; return KR_OK; }
long kr_serve_graph_replays(const kr_serve* s) { return s ? s->graph_replays : 0; }

int kr_serve_sample(kr_serve* s, int row, float temperature, int top_k, float top_p, uint64_t rng_seed, int* token_out) {
    if (!s || !token_out) return kr_fail(KR_ERR_VALUE, "null argument");
    if (row < 0 || row >= s->last_want) return kr_fail(KR_ERR_VALUE, "row %d of the last step's %d", row, s->last_want);
    KR_HIP(hipSetDevice(s->device));
    const int V = s->c.vocab;
    const size_t tb = kr_sampler_temp_bytes(V);
    if (s->s_keys.ensure((size_t)V * 8) || s->s_sorted.ensure((size_t)V * 8) || s->s_temp.ensure(tb) || s->s_probs.ensure((size_t)V * 4) || s->s_rng.ensure(8) ||
        s->s_tok.ensure(4) || s->s_seen.ensure(((size_t)V + 31) / 32 * 4) || s->s_row.ensure((size_t)V * 4))
        return kr_fail(KR_ERR_HIP, "sampler scratch");
    if (!(temperature > 0.0f)) return kr_fail(KR_ERR_VALUE, "temperature %g: greedy decoding reads the step's argmax", (double)temperature);
    KR_HIP(hipMemsetAsync(s->s_seen.p, 0, ((size_t)V + 31) / 32 * 4, s->st));
    if (rng_seed == 0) rng_seed = 0x9E3779B97F4A7C15ull;
    KR_HIP(hipMemcpyAsync(s->s_rng.p, &rng_seed, 8, hipMemcpyHostToDevice, s->st));
    KR_HIP(hipMemcpyAsync(s->s_row.p, (const float*)s->logits.p + (size_t)row * V, (size_t)V * 4, hipMemcpyDeviceToDevice, s->st));   // the sampler scales in place
    if (kr_launch_sample((float*)s->s_row.p, V, temperature, top_k, top_p, 0.0f, (uint32_t*)s->s_seen.p, (uint64_t*)s->s_keys.p, (uint64_t*)s->s_sorted.p, s->s_temp.p, tb,
                         (float*)s->s_probs.p, (uint64_t*)s->s_rng.p, (int*)s->s_tok.p, s->st))
        return kr_fail(KR_ERR_HIP, "sampler launch failed");
    KR_HIP(hipMemcpyAsync(token_out, s->s_tok.p, 4, hipMemcpyDeviceToHost, s->st));
    KR_HIP(hipStreamSynchronize(s->st));
    return KR_OK;
}

}  // extern "C"
