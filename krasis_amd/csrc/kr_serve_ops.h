// kr_serve_ops.h -- launch wrappers of the batched serving kernels (kr_serve_ops.hip, kr_serve_gemm.hip).
//
// One step of the serving store is a ragged batch: T tokens of several requests, each with its own cache slot and position.  Weights, GEMM inputs
// and cache rows have the storage type of the store (bf16 or f32: `f32` flag below); positions, angles, norms, router, scores, softmax weights and
// the residual stream are f32 in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

// ---- GEMM: C[M, N] (f32) = A[M, K] x W[N, K]^T, storage type bf16 (matrix cores, f32 accumulation) or f32 (plain fused multiply-adds)
struct KrSvGemm {
    const void* A; int lda;          // rows of K storage elements
    const void* W; size_t w_stride;  // [N, K] row-major; grouped: matrix g at W + g * w_stride elements
    float* C; int ldc;
    int M, N, K;
    const int* a_rows;               // optional: problem row r reads A row a_rows[r]
    const int* seg;                  // grouped: [n_groups + 1] row offsets on the device (rows of group g are [seg[g], seg[g + 1])); null = one matrix
    const int* row_group;            // grouped: [M] group of every row (the small-M form reads it)
    int n_groups;
    // small-M form only (kr_sv_gemm_small): A is not read but formed on the fly as the gated activation of act_gu [M, act_ld] f32 (gate at column k, up at
    // column K + k), rounded to the storage type -- the down projection of a feed-forward without a launch and a buffer for the activation
    const float* act_gu; int act_ld, act_kind; float act_limit, act_alpha;
    const int* c_rows;               // optional: problem row r writes C row c_rows[r] (a grouped problem whose rows return to their own order)
    int c_storage;                   // != 0: C holds the storage type (bf16 in a bf16 store) instead of f32 -- the output feeds another GEMM as it is
    int rowwise_upto;                // grouped problems: the wave-per-column form up to this many rows (0 = the default of 64)
};
void kr_sv_gemm(const KrSvGemm& g, bool f32, hipStream_t st);
bool kr_sv_gemm_small(const KrSvGemm& g);      // true: kr_sv_gemm takes the wave-per-column form for this problem (and honours act_gu)

enum { KR_SV_NORM_LAYER = 0, KR_SV_NORM_RMS = 1 };
enum { KR_SV_ACT_GELU_TANH = 0, KR_SV_ACT_CLAMPED_SWIGLU = 1, KR_SV_ACT_SILU = 2, KR_SV_ACT_RELU2 = 3 /* un-gated: relu(x)^2 of the first F columns; no up columns */ };

// x[t] = table[tokens[t]]; with h_out also the row in the storage type (the first sublayer's input in a design without input norms)
// scale: the row is multiplied by it (1 = as it is)
// table2 / rows2: optional second table whose row rows2[t] is added as it is (a hashed pair-of-tokens embedding)
void kr_sv_embed(const void* table, bool f32, const int* tokens, float* x, void* h_out, int T, int width, float scale, const void* table2, const int* rows2, hipStream_t st);
// the stream itself: x[t] += add (optional [width]); then, with w, either x[t] <- norm(x[t]) * w (in_place: the normed row IS the stream) or
// out[t] = norm(x[t]) * w in the storage type (the next sublayer's input).  One workgroup per row, the row held in LDS.
void kr_sv_stream_norm(float* x, const float* add, const float* w, const float* b, bool in_place, void* out, bool out_f32, int T, int width, float eps, int kind, int groups,
                       hipStream_t st);
// Short causal convolution over a request's positions on C channels of a projection's output:
//   y[t][c] = act(cb[c] + sum_j w[c][j] u(position(t) - taps + 1 + j)[c]),  u = in + in_bias, zeros before position 0.
// u of a position comes from this step's rows when the request's portion holds it, else from the request's ring state[slot][position % (taps - 1)][C];
// kr_sv_chan_conv_save (a launch of its own, after the convolution has read the ring) keeps the last taps - 1 rows u of every portion.
struct KrSvChanConv {
    const float* in; int ld_in;      // [T, ld_in] f32, the C channels start at `in`
    const float* in_bias;            // [C] or null: joins the input before the convolution (a projection's bias)
    const float* w; int taps;        // [C, taps] f32, the last column is the current token's
    const float* cb;                 // [C] or null: the convolution's own bias
    int act;                         // 0 none, 1 silu
    float* out; int ld_out;          // [T, ld_out] f32 (not `in`)
    float* state;                    // [slots][taps - 1][C]
    const int* slot; const int* pos; int T, C;
    const int* ent_off; int n_entries;
};
void kr_sv_chan_conv(const KrSvChanConv& c, hipStream_t st);
void kr_sv_chan_conv_save(const KrSvChanConv& c, hipStream_t st);
// logits <- logits * scale
void kr_sv_scale(float* p, size_t n, float scale, hipStream_t st);
// out[r] = norm(x[rows ? rows[r] : r]) * w (+ b): two passes over the row, f32; out in the storage type.  groups > 1: the row is normed in that many equal
// consecutive parts, each by its own statistics.  out32: optional f32 copy of the normed row (the input of a convolution over positions)
void kr_sv_norm(const float* x, const int* rows, const float* w, const float* b, void* out, bool out_f32, int R, int width, float eps, int kind, int groups, float* out32,
                hipStream_t st);
// Input convolution over a request's positions: hc[t] = h[t] + sum_j w[:, j] h(position(t) - taps + 1 + j), channel by channel, zeros before position 0.
// h of a position comes from this step's rows (h32 [T, width]: the rows of one request stand together, in order) or, for positions before the
// step's portion, from the request's state: state[slot][position % (taps - 1)][width] f32.  kr_sv_canon_save (any launch after the convolution) keeps
// the last taps - 1 rows of every portion there.
struct KrSvCanon {
    const float* h32; const float* w; int taps;      // w [width, taps]
    float* state;                                    // [slots][taps - 1][width]
    const int* slot; const int* pos; int T, width;
    void* out;                                       // [T, width] storage type
};
void kr_sv_canon(const KrSvCanon& c, bool f32, hipStream_t st);
// cos / sin of pos * inv_freq for every token of the step: cs[t][i] = mult * (cos, sin), the angle formed in double
void kr_sv_rope_table(const int* pos, const double* inv_freq, float2* cs, int T, int half, float mult, hipStream_t st);

struct KrSvAttn {
    float* qkv; int ldq;             // [T, ldq] f32: q heads, then k heads, then v heads (k / v absent when the layer borrows another layer's cache)
    int heads, kv_heads, dim, vdim, rot_dims, rot_interleaved, unit_norm, own_kv;
    const float* q_norm_w; const float* k_norm_w;   // [dim] each: unit_norm == 2 (weighted, before the rotation)
    float eps, scale;
    int window;                      // 0 = every earlier position
    int chunk;                       // > 0: only the keys of the query's own block of `chunk` positions (counted from position 0 of the request)
    const float* slopes;             // [heads] or null: score -= slopes[h] * (query position - key position)
    int v_mix; const float* v_lambda; float* v_first;   // 1: values also kept in v_first [T, kv_heads * vdim]; 2: v <- (1 - *v_lambda) v + *v_lambda v_first
 // ---- biases, whole-projection norm, values that are the un-normed keys, capped scores, gated output
    const float* q_bias; const float* k_bias;        // [heads * dim], [kv_heads * dim] or null: added before anything else
    const float* inv_rms;            // unit_norm == 3: [T, 2] 1 / rms of the whole q and the whole k row (kr_sv_qk_rms), weights q_norm_w [heads * dim], k_norm_w [kv_heads * dim]
    float* inv_rms_out;              // where kr_sv_qk_rms writes them
    int v_from_k;                    // the value rows of the cache are the key rows before their norm (no v block in qkv)
    float softcap;                   // > 0: score <- softcap * tanh(score / softcap) before the distance bias
    const float* out_gate; int ld_gate;   // [T, ld_gate] f32 or null: head h's output is multiplied by sigmoid(out_gate[t][h])
    const float* v_bias;             // [kv_heads * vdim] or null: joins the values before they are cached
    int gate_elem;                   // out_gate holds one logit per output coordinate ([T, ld_gate] with heads * vdim columns) instead of one per head
    float out_scale;                 // the output is multiplied by it before it is rounded (0 reads as 1)
    int out_ld;                      // row stride of `out` in elements (0: heads * vdim) -- the output may be the leading columns of a wider row
    const float* sink;               // [heads] or null
    const float2* cs;                // rope table of the step for this layer's rotation
    void* kpool; void* vpool;        // [pages][page_tokens][ldk | ldv] storage type; head g at g * dim | g * vdim of a row (vpool may be kpool: values that are a
    int ldk, ldv;                    //   leading part of the key row)
    const int* page_table; int table_ld;   // [slots][table_ld]
    const int* slot; const int* pos; // per token
    int page_tokens, T;
    void* out;                       // [T, heads * vdim] storage type
    int nsplit;                      // >= 1: workgroups that share a token's keys (few tokens: more of the chip per token); > 1 needs the two buffers below
    float* part_ml; float* part_acc; // [T][heads][nsplit][2] running (maximum, denominator), [T][heads][nsplit][vdim] unnormalised sums
    int tq;                          // set by the launcher of the matrix-instruction form: tokens per workgroup
};
// how many ways to split: fills the chip when the step has few tokens; max_visible = most keys any token of the step sees in this layer
int kr_sv_attention_splits(int T, int heads, int kv_heads, int dim, int vdim, int ldk, int ldv, bool f32, int max_visible);
void kr_sv_qk_rms(const KrSvAttn& a, hipStream_t st);                 // unit_norm == 3: the two whole-row statistics of every token
void kr_sv_qk_prep(const KrSvAttn& a, bool f32, hipStream_t st);      // biases, rotation, unit norm, cache append
void kr_sv_attention(const KrSvAttn& a, bool f32, hipStream_t st);   // windowed softmax with an optional sink over the paged cache

// group-limited top-k router on logits z (rows `ld` floats apart, `parts` column blocks of E that are added): softmax over all experts, the best `keep` of
// `groups` groups (a group's score = its largest), `top` experts among them; weights = the softmax scores (renorm != 0: divided by their sum).
// The logits come from kr_sv_gemm: an f32 store multiplies by the f32 gate; a bf16 store by the gate as two bf16 terms (hi + lo rows), which
// carries 16 bits of the gate's mantissa through the matrix cores.
// bias [E] or null: bias_mode 1 joins the logits before anything else; 2 joins the scores for the choice of groups and experts only (the weights are the
// scores without it).  score_kind 0: softmax over all experts, 1: sigmoid of every logit.  group_kind 0: a group's score is its largest choice score,
// 1: the sum of its two largest.  Experts outside the kept groups cannot be chosen, whatever their score.  renorm: weights / (their sum + 1e-20).
void kr_sv_router_select(const float* z, int ld, int parts, const float* bias, int bias_mode, int score_kind, int group_kind, int T, int E, int top, int groups, int keep,
                         int renorm, int* ids, float* wts, hipStream_t st);
// rows of every expert: seg[E + 1], src_row[T * top] (token of sorted row), row_group[T * top], pair_pos[T * top] (sorted row of (token, slot))
void kr_sv_moe_sort(const int* ids, int T, int top, int E, int* counts, int* seg, int* cursor, int* src_row, int* row_group, int* pair_pos, hipStream_t st);
// gu rows `ld` floats apart (gate at [0, F), up at [F, 2F)) -> y [M, F] storage type
void kr_sv_act(const float* gu, int ld, void* y, bool f32, int M, int F, int kind, float limit, float alpha, hipStream_t st);
// y[t] = mix[t] + (dense[t] + shared[t] + sum_s wts[t][s] * rows[pair_pos[t][s]]) (null terms are skipped); with post_w, y <- norm(y) * post_w (+ post_b);
// x[t] += mult * y[t].  With h_out the NEW row goes there in the storage type by the same launch: normed with norm_w (+ norm_b) -- the next sublayer's
// input -- or, without norm_w, as it is.
struct KrSvResidual {
    float* x; const float* mix; const float* dense; const float* shared; const float* rows; const int* pair_pos; const float* wts; int top;
    const float* post_w; const float* post_b; float mult;
    const float* norm_w; const float* norm_b; void* h_out;
    int T, width, kind; float eps;
    int groups;                      // > 1: both norms work on that many equal parts of the row
    float* h32_out;                  // optional f32 copy of the handed-on row
    const float* gate; int ld_gate; const float* gate_b;   // y <- y * sigmoid(gate[t] + gate_b) element by element, before it joins x (null = no gate)
    const float* mix_bias;           // [width] or null: added to mix (the output projection's bias)
    // the input convolution's state: rows of h32_in that are among the last canon_keep of their request's portion go to canon_state[slot][pos % canon_keep]
    const float* h32_in; float* canon_state; int canon_keep; const int* slot; const int* pos;
};
void kr_sv_residual_norm(const KrSvResidual& r, bool out_f32, hipStream_t st);

// ---- latent mixer (queries and keys / values through low-rank latents; the cache row is [latent | rotated shared key part])
struct KrSvLatent {
    const float* dz; int ld;         // [T, ld] f32: W_dq h [q_rank] | W_dkv h [kv_rank + rot]
    int q_rank, kv_rank, rot, heads, dim;
    const float* dq_norm_w; const float* dkv_norm_w; float eps;
    const float2* cs;                // rotation table of the step [T, rot / 2]
    void* cq;                        // out [T, q_rank] storage type: rms(W_dq h) * w
    void* pool; const int* page_table; int table_ld; const int* slot; const int* pos; int page_tokens, T;    // cache rows [kv_rank + rot] storage type
};
// normed query latent -> cq; normed key / value latent and the rotated shared key part -> the cache row of (slot, position)
void kr_sv_latent_prep(const KrSvLatent& a, bool f32, hipStream_t st);
// q2 [T, heads, dim + rot] f32 (W_uq c_q): the plain part -> qn [T, heads, dim] storage type (to be folded into the latent space by a GEMM), the rotated
// part, turned, -> qe [T, heads, kv_rank + rot] f32 at column kv_rank
void kr_sv_latent_q(const KrSvLatent& a, const float* q2, void* qn, float* qe, bool f32, hipStream_t st);
// rows of a problem grouped by head over [T, heads, *] arrays: seg[h] = h * T, rows[h * T + t] = t * heads + h, group[h * T + t] = h
void kr_sv_head_rows(int T, int heads, int* seg, int* rows, int* group, hipStream_t st);

// ---- recurrent mixers: per head a matrix state S [dim, vdim] (f32) carried from token to token of a request
//   retention: S_t = decay_h S_(t-1) + k_t v_t^T,                                   o_t = S_t^T q_t
//   mlstm:     m_t = max(f_t + m_(t-1), i_t); S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T; n_t alike with k_t alone;
//              o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6);  i = cap(z_i + b_i), f = logsigmoid(cap(z_f + b_f)), cap(z) = gate_cap tanh(z / gate_cap)
// then o / rms(o) per head (* norm_w) * act(g) -> out in the storage type (act: silu for retention, sigmoid for mlstm).
// The state of request slot s: S at state + s * state_stride as [heads][vdim][dim]; normaliser and maximum at nm + s * nm_stride as
// [heads][vdim blocks of 16][dim + 4] (every block of value columns keeps its own copy, so no two workgroups share a word).  A portion that starts at
// position 0 starts from zeros whatever the slot held.
//   gla (4):   S_t = diag(a_t) S_(t-1) + k_t v_t^T, a_t = exp(log sigmoid(gz_t + gz_bias) * inv_tau) per key channel (gz [T, gz_ld], heads x dim)
//   ssd (5):   S_t = exp(-exp(a_log_h) dt_t) S_(t-1) + dt_t k_t v_t^T with dt_t = softplus(dtz_t[h] + dt_bias[h]); q, k of head h are those of group
//              h / qk_group (C and B), v the head's x; the skip term and everything after it belong to kr_sv_ssd_out
// Kinds 4 and 5 read q, k, v through qsrc / ksrc / vsrc (rows src_ld floats apart); the scan form only.
struct KrSvLin {
    int kind;                        // KR_SERVE_MIX_RETENTION (2) | KR_SERVE_MIX_MLSTM (3) | KR_SERVE_MIX_GLA (4) | KR_SERVE_MIX_SSD (5)
    const float* qsrc; const float* ksrc; const float* vsrc; int src_ld, qk_group;      // kinds 4, 5
    const float* gz; int gz_ld; const float* gz_bias; float inv_tau;                     // kind 4
    const float* dtz; int dtz_ld; const float* dt_bias; const float* a_log;              // kind 5
    int norm_shared;                 // norm_w is [vdim], shared by the heads
    int prepped;                     // kr_sv_lin_chunked: z already holds q, k as the block launches read them and tok the log decays (kr_sv_ssd_expand)
    float* z; int ld;                // [T, ld] f32: q [heads * dim] | k [heads * dim] | v [heads * vdim] | g [heads * vdim] | (mlstm) z_i [heads] | z_f [heads]
    int heads, dim, vdim, rot_dims;
    const float2* cs;                // rotation table of the step [T, rot_dims / 2] (pairs (i, i + rot_dims / 2))
    float q_scale, k_scale;
    const float* decay;              // [heads] (retention)
    const float* i_bias; const float* f_bias; float gate_cap;     // mlstm
    float* state; size_t state_stride; float* nm; size_t nm_stride;
    const int* ent_off; const int* ent_slot; int n_entries;       // rows [ent_off[e], ent_off[e + 1]) belong to slot ent_slot[e]
    const int* pos; int T;
    float* o;                        // [T, heads * vdim] f32 scratch
    const float* norm_w; float eps;  // [heads * vdim] or null
    void* out;                       // [T, heads * vdim] storage type
    // chunked form (prompt portions): blocks of 64 tokens counted from the start of every entry's portion; entry e owns the blocks
    // [ent_chunk0[e], ent_chunk0[e + 1])
    const int* ent_chunk0; int n_chunks;
    float4* tok;                     // [T, heads]: per token (u = F - m, w = b - F, g = exp(F + m_start - m), exp(-m)); F = log decay summed from the block's start
    float* sbuf; float* nbuf;        // [n_chunks, heads, dim, vdim] / [n_chunks, heads, dim]: state and normaliser at every block's start
    float* cmeta;                    // [n_chunks, heads, 4]: a block's last F, its last prefix maximum of b - F, the running maximum at its start
};
// token by token, the state in registers: decode steps and short portions
void kr_sv_lin_scan(const KrSvLin& a, hipStream_t st);
// prompt portions in blocks of 64 tokens on the f32 matrix instruction (rotation and scales applied to q / k in place first): within a block
// o_t = g_t S_start^T q_t + sum_(s <= t) exp(u_t + w_s) (q_t . k_s) v_s, and S_end = g_last S_start + sum_s exp(u_last + w_s) k_s v_s^T; a short serial
// launch carries S from block to block, the outputs of all blocks are formed in parallel.  Same state layout as kr_sv_lin_scan.
// kinds 4 and 5, prompt portions: a workgroup per (request, head, 8 value columns), the rows of S spread over thirty-two lanes per column, tokens staged
// sixteen at a time through two LDS buffers.  For kind 4 the launcher first turns a.gz (written by the caller, logits) into the decays, in place.
bool kr_sv_lin_scan_wide_fits(int kind, int dim);
void kr_sv_lin_scan_wide(const KrSvLin& a, hipStream_t st);
bool kr_sv_lin_chunked_fits(int dim, int vdim);
void kr_sv_lin_chunked(const KrSvLin& a, hipStream_t st);
// the state-space recurrence (kind 5 fields of `a`) written as a retention with a decay per token: z_out [T, ldz] = per head [q = C | k = dt B | v = x] in
// the recurrent mixers' layout, a.tok[t][head].x = the token's log decay.  Follow with kr_sv_lin_chunked on a kind-2 description with prepped = 1.
void kr_sv_ssd_expand(const KrSvLin& a, float* z_out, int ldz, hipStream_t st);
void kr_sv_lin_out(const KrSvLin& a, bool f32, hipStream_t st);
// the selective state-space mixer after its scan: y = (o + D_h x) * silu(z), rms-normed in `groups` equal parts of the inner row, times w, times scale,
// rounded to the storage type at out[t * out_ld + c]
struct KrSvSsdOut {
    const float* o;                  // [T, inner] f32 (the scan's output)
    const float* x; int ld_x;        // the convolved x rows
    const float* z; int ld_z;        // the gate's pre-activation
    const float* D;                  // [heads]
    const float* w;                  // [inner]
    int heads, vdim, groups; float eps, scale;
    void* out; int out_ld; int T;
};
void kr_sv_ssd_out(const KrSvSsdOut& a, bool f32, hipStream_t st);
void kr_sv_argmax(const float* logits, int R, int vocab, int* out, hipStream_t st);
// uniform values in [-amp, amp) from a counter hash of (seed, element); amp = 0 writes zeros
void kr_sv_fill_uniform(void* p, bool f32, size_t n, uint64_t seed, float amp, hipStream_t st);
