// k_layered.hpp — launchers of the layered-model kernels (k_layered.hip).  Host functions take
// a stream, never allocate or synchronise, and return 0 or an error with qie_last_error() text.
#pragma once

#include "qie_common.hpp"

namespace qie {
namespace lay {

// y[m, n] = sum_k A[m, k] W[n, k] (+ batch z: A + z sA, W + z sW, Y + z sY).  A fp32, rounded to
// bf16 on load when round_a; W fp32 or bf16 words; Y fp32.  grp_off (device, batch + 1 entries):
// batch z covers rows [grp_off[z], grp_off[z + 1]) of A and Y (M is then the largest row count a
// group can have).  Three kernels by shape: up to 32 rows a column-per-wave kernel, many rows of a
// bf16 model (mfma) MFMA tiles from memory, else 64 x 64 fp32 tiles through LDS; an element's sum
// never depends on what else the launch holds, only on which of the three ran.
struct LinearP {
    const float* A;
    int64_t lda;
    const void* W;
    int64_t ldw;
    float* Y;
    int64_t ldy;
    int M, N, K, batch;
    int64_t sA, sW, sY;
    int round_a;
    const int32_t* grp_off;
    int mfma;   // bf16 weights, many rows: the direct MFMA kernel may take the product (batched / grouped forms)
};
int linear(const LinearP& p, bool w_f32, hipStream_t st);

// Paged latent cache: page p at pool + p * page_stride elements; inside a page the rows of one
// caching layer start at layer_off and are D = R + rot wide: [c (R) | rotated shared key (rot)].
// Token t of slot s is row t % page_tokens of page table[s * max_pages + t / page_tokens].
struct LatentCache {
    void* pool;
    int64_t page_stride;
    const int32_t* table;
    int page_tokens, max_pages;
};

struct LatentPostP {
    float* proj;          // [T][ld]: q heads, then (own_kv) the compressed row and the shared key part
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, dim, rot, rot_dims, R, own_kv;
    const float* norm_w;  // [R]
    float eps;
    const float* rope_cos;   // [positions][rot_dims / 2]
    const float* rope_sin;
    LatentCache cache;
    int64_t layer_off;
    int interleaved;      // bf16 caches: also write the key-interleaved copy of c that follows the rows
    int rot_layout;       // 0: coordinate i turns with i + rot_dims / 2; 1: 2i with 2i + 1
    const float* kv;      // own_kv: where the compressed row and the shared key part are read from
    int64_t kv_ld;        //   ([T][kv_ld], columns 0 .. R + rot); null: the projection row after the q heads
};
int latent_post(const LatentPostP& p, bool cache_f32, int T, hipStream_t st);

struct LatentAttnP {
    const float* q_abs;   // [T][heads][R]
    const float* proj;    // rotated query parts are read from the projection rows
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, dim, rot, R, window;
    float scale;
    LatentCache cache;
    int64_t layer_off;
    float* out;           // [T][heads][R]
};
int latent_attention(const LatentAttnP& p, bool cache_f32, int T, hipStream_t st);

// The matrix-core form (k_latent_attn.hip; bf16 cache rows followed, per caching layer and page,
// by the key-interleaved copy of c: element ((t % page_tokens) / 4 * R + r) * 4 + t % 4).  A row
// group is up to 16 (token, head) rows of consecutive tokens of one slot: {first packed row,
// tokens, first head, heads per token}.  S splits over the keys; part_o [groups * S][16][R] and
// part_ml [groups * S][16][2] are scratch.
struct LatentAttnMfmaP {
    const float* q_abs;
    const float* proj;
    int64_t ld;
    const int32_t* row_slot;
    const int32_t* row_pos;
    const int4* groups;
    int n_groups, S;
    int heads, dim, rot, R, window;
    float scale;
    LatentCache cache;
    int64_t layer_off;
    float* part_o;
    float* part_ml;
    float* out;           // [T][heads][R]
};
// Row groups a wave takes together: the group list of a step holds, per entry, a multiple of
// kLatentQG groups (padded with empty groups {row, 0, 0, 1}), and consecutive groups of a unit
// belong to one slot.
constexpr int kLatentQG = 1;   // 2 measured slower at kv_rank 256 (one wave per SIMD), and spills at 512
bool latent_attention_mfma_fits(int R, int rot);
int latent_attention_mfma(const LatentAttnMfmaP& p, hipStream_t st);

// ------------------------------------------------------------------ grouped-query attention
// (k_mixers.hip)  Paged K / V rows: inside a page the K rows of one cache region start at k_off
// and are kv_heads * dim wide, its V rows at v_off, kv_heads * vdim wide (LatentCache names the
// pool, its block table and the page geometry).
//
// gqa_post: per row of the fused projection, every query and key head is RMS-normed over dim
// (qk_norm: 0 no, 1 with the weight qn_w / kn_w, 2 without one), its first rot_dims coordinates
// are turned by the row's position (layout 0: i with i + rot_dims / 2; 1: 2i with 2i + 1); queries
// go back in place, keys to the cache.  Values: v_col < 0 caches the key as projected (before its
// norm) as the value; else W_v's columns, turned over all vdim coordinates when rot_values.
struct GqaPostP {
    float* proj;
    int64_t ld;
    int q_col, k_col, v_col;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, kv_heads, dim, vdim;
    int qk_norm;
    const float* qn_w;
    const float* kn_w;
    float eps;
    int rot_dims, rot_layout;
    const float* rope_cos;    // [positions][rot_dims / 2]
    const float* rope_sin;
    int rot_values;
    const float* vrope_cos;   // [positions][vdim / 2]
    const float* vrope_sin;
    LatentCache cache;
    int64_t k_off, v_off;
    int v_transposed;         // V rows of a page stored [kv_heads][vdim][page_tokens]
    // q_temp_every > 0: the normed query is multiplied by 1 + q_temp_coef * ln((pos + 1) / every + 1),
    // the division rounded down
    int q_temp_every;
    float q_temp_coef;
    const float* q_bias;      // [heads * dim] / [kv_heads * dim] or null: added to q / k as they leave the projection
    const float* k_bias;      //   (a key cached as the value carries its bias)
};
int gqa_post(const GqaPostP& p, bool cache_f32, int T, hipStream_t st);

// Softmax attention of every (row, head) over the keys its mask lets it see (mask 0: all j <= i;
// 1: the last mask_size; 2: those with j / mask_size == i / mask_size); score = q.k * scale
// - r1[h] * ln(1 + r2[h] * (i - j)) when r1 is set.  rot_values: the weighted sum is turned back
// by the row's position.  The result times out_scale goes to out[t * ld_out + out_col + h * vdim
// ...] (and its bf16 image).
struct GqaAttnP {
    const float* proj;
    int64_t ld;
    int q_col;
    const int32_t* row_slot;
    const int32_t* row_pos;
    int heads, kv_heads, dim, vdim;
    int mask, mask_size;
    float scale;
    const float* r1;
    const float* r2;
    int rot_values, rot_layout;
    const float* vrope_cos;
    const float* vrope_sin;
    LatentCache cache;
    int64_t k_off, v_off;
    int v_transposed;
    float out_scale;
    float* out;
    uint16_t* out_bf;
    int64_t ld_out;
    int out_col;
    const float* slopes;      // [heads] or null: the score also loses slopes[h] * (i - j)
    const float* pb;          // [heads] or null; set: a visible key's weight is sigmoid(score + pb[h]),
                              // and the weights of a row are used as they are (no softmax)
    int gate_col;             // >= 0: head h's result times sigmoid(proj[t * ld + gate_col + h])
    int gate_elem;            // with gate_col: one gate per coordinate, proj[t * ld + gate_col + h * vdim + c]
    const float* sink;        // [heads] or null: exp(sink[h]) joins the softmax denominator (no key, no value)
};
int gqa_attention(const GqaAttnP& p, bool cache_f32, int T, hipStream_t st);
// The matrix-core form for bf16 caches whose V rows are stored transposed (v_transposed: inside a
// page [kv_heads][vdim][page_tokens], so that 4 keys of one value coordinate are one 8-byte load;
// page_tokens a multiple of 32), dim a multiple of 32 and vdim of 16, both up to 256.  A wave takes
// up to 16 (token, head) columns of one slot that share a key head: 16 consecutive tokens of one
// head, or - for groups of few tokens, see pack - the heads of one key head per token.  groups: {first
// packed row, tokens (<= 16), slot, first position}.  S > 1 splits every wave's keys S ways
// (decoding: few columns, many keys); the partial sums meet in a second pass.  part_o
// [groups * tiles * S][16][vdim], part_ml [...][16][2] floats of scratch (tiles = 4 * ceil(heads / 4)).
struct GqaAttnMfmaP {
    GqaAttnP a;
    const int4* groups;
    int n_groups, S;
    float* part_o;
    float* part_ml;
    // 1: groups of few tokens pack the heads of a key head into a wave's columns, every wave loads
    // its own fragments (head ratios that are no multiple of 4); 0: one head per wave, the four
    // waves of a workgroup share their key head's tiles through LDS (ratios that are)
    int pack;
};
bool gqa_attention_mfma_fits(int dim, int vdim, int page_tokens);
int gqa_attention_mfma(const GqaAttnMfmaP& p, hipStream_t st);

// ------------------------------------------------------------------ gated linear recurrence
// Per entry {first packed row, rows, slot, first position} and head: S [dim][vdim] (fp32, at
// state + slot * slot_stride + state_off) runs through the entry's rows in order,
// S = diag(f) S + (1 - f) v^T, o = S^T q, with q = silu(proj[q_col ...]),
// f = lower + (1 - lower) * sigmoid(proj[f_col ...] + f_bias); an entry whose first position is 0
// starts from S = 0.  Raw o -> out [T][heads * vdim].
struct GatedScanP {
    const float* proj;
    int64_t ld;
    int q_col, f_col, v_col;
    const int4* entries;
    int n_entries;
    int heads, dim, vdim;
    const float* f_bias;
    const float* lower;
    float* state;
    int64_t slot_stride, state_off;
    float* out;
    // mode 0: the recurrence itself (state read unless the entry starts at position 0, advanced,
    // written back); decay (optional) receives the product of the entry's gates, [entries][heads][dim].
    // mode 1: the state is only read, every row's q is scaled by the product of the gates from the
    // entry's first row to this row, and out receives S^T q: the share of an incoming state in the
    // outputs of rows that were scanned from a zero state (the caller adds the two).
    int mode;
    float* decay;
};
int gated_scan(const GatedScanP& p, hipStream_t st);
// Long entries in pieces: `chunks` lists pieces {first packed row, rows, piece index, 0} in entry
// order, `spans` one {first piece, pieces, slot, first position} per entry.  gated_scan (mode 0)
// over the pieces from zero states gives piece-local outputs, end states s_loc [pieces][heads *
// dim * vdim] and gate products; gated_carry walks an entry's pieces in order (s_in[c] = state
// entering piece c, starting from the slot's state or zero; the slot's state = what leaves the
// last piece); gated_scan (mode 1) over the pieces with s_in gives the incoming states' share.
// Same sums as the row-by-row recurrence up to fp32 rounding.
struct GatedCarryP {
    const int4* spans;
    int n_spans;
    int heads, dim, vdim;
    const float* s_loc;
    const float* decay;
    float* s_in;
    float* state;
    int64_t slot_stride, state_off;
};
int gated_carry(const GatedCarryP& p, hipStream_t st);
// out[t, out_col + h * vdim + c] = scale * o[t, h, c] / sqrt(mean_c o^2 + eps) * w[c], o = o1 + o2 when o2
// ------------------------------------------------------------------ minGRU
// Per entry {first packed row, rows, index, first position} and channel c < n: with
// z = sigmoid(proj[z_col + c] + z_b[c]), u = proj[x_col + c] + x_b[c], cand = u >= 0 ? u + 1/2 :
// sigmoid(u), the state runs through the entry's rows in order, S = (1 - z) S + z cand, and
// out[row, c] = S * silu(proj[g_col + c]) (with its bf16 image).  fp32 throughout.
// init: the state an entry starts from, at init + index * init_stride (+ init_off); null, or (when
// init_if_pos) an entry whose first position is 0: zero.  end / decay (optional, same addressing
// with end_stride): the state after the entry's last row, the product of its (1 - z).  out may be
// null (a pass that only wants end and decay).
struct MinGruScanP {
    const float* proj;
    int64_t ld;
    int z_col, x_col, g_col;
    const float* z_b;
    const float* x_b;
    const int4* entries;
    int n_entries, n;
    const float* init;
    int64_t init_stride, init_off;
    int init_if_pos;
    float* end;
    float* decay;
    int64_t end_stride, end_off;
    float* out;
    uint16_t* out_bf;
    int64_t ld_out;
};
int mingru_scan(const MinGruScanP& p, hipStream_t st);
// Long entries in pieces (lists as for gated_carry): s_in[c] = the state entering piece c, from the
// slot's state (or zero at position 0) through S <- decay[c] S + s_loc[c]; the slot's state = what
// leaves the entry's last piece.
struct MinGruCarryP {
    const int4* spans;
    int n_spans, n;
    const float* s_loc;
    const float* decay;
    float* s_in;
    float* state;
    int64_t slot_stride, state_off;
};
int mingru_carry(const MinGruCarryP& p, hipStream_t st);

// gate (optional, [T][heads * vdim]): the result is also multiplied by sigmoid(gate[t, h * vdim + c])
int head_norm_rows(const float* o, const float* o2, const float* w, float eps, float scale, int heads, int vdim, int T, float* out,
                   uint16_t* out_bf, int64_t ld_out, int out_col, hipStream_t st, const float* gate = nullptr);

// ------------------------------------------------------------------ residual streams (k_streams.hip)
// n residual rows per token, X + s * plane (rows of W).  With y (a sublayer's result, [T][W]) the rows
// are replaced, all at once from the old ones, by x_t = sum_s mix[s * n + t] x_s + out[t] y.  With `in`
// the read-out u = sum_s in[s] x_s of the (new) rows is normed, h = u / sqrt(mean(u^2) + eps) *
// (w_one + wn), with its bf16 image.  sum (optional) receives the plain sum of the (new) rows.
struct StreamStepP {
    float* X;
    int64_t plane;
    int n;
    const float* y;
    const float* mix;
    const float* out;
    const float* in;
    const float* wn;
    float w_one, eps;
    float* h;
    uint16_t* h_bf;
    float* sum;
    int T, W;
};
int stream_step(const StreamStepP& p, hipStream_t st);

// Causal convolution over time per channel on the packed rows of a step: out[t, c] =
// (residual ? in[t, c] : 0) + sum_j w[c * taps + j] in[t - (taps - 1 - j), c], then silu when asked.
// Rows before an entry's first come from the slot's state ([taps - 1][C] floats at state + slot *
// slot_stride + state_off: the inputs at the taps - 1 positions before the entry, oldest first), rows
// before position 0 are zero.  row_k: a row's index inside its entry.  causal_conv_state moves the
// state on by the step's entries {first packed row, rows, slot, first position}; run it after
// causal_conv (which reads the old state) and before `in` is overwritten.
struct CausalConvP {
    const float* in;
    int64_t ld_in;
    int col, C, taps;
    const float* w;
    const int32_t* row_slot;
    const int32_t* row_pos;
    const int32_t* row_k;
    float* state;
    int64_t slot_stride, state_off;
    int residual, silu;
    float* out;
    int64_t ld_out;
    uint16_t* out_bf;
    const int4* entries;
    int n_entries;
};
int causal_conv(const CausalConvP& p, int T, hipStream_t st);
int causal_conv_state(const CausalConvP& p, hipStream_t st);
// Both in order; steps of at most kConvFusedRows rows in one launch (a thread per entry and channel)
constexpr int kConvFusedRows = 64;
int causal_conv_advance(const CausalConvP& p, int T, hipStream_t st);
// out[t, c] = in[t, col + c] / sqrt(mean_c in^2 + eps) * (w_one + w[c]), c < n (out may be in + col)
int rms_rows(const float* in, int64_t ld_in, int col, int n, const float* w, float w_one, float eps, float* out, int64_t ld_out,
             uint16_t* out_bf, int T, hipStream_t st);

// ------------------------------------------------------------------ gated delta rule (k_delta.hip)
// qkv [T][ld_qkv]: q (G heads of dim), k (G x dim), v (H x vdim) after their convolutions.  delta_prep,
// in place: q and k heads to unit length (x / sqrt(sum x^2 + 1e-6)), q also times dim^(-1/2);
// proj[t, b_col + h] = sigmoid of itself; a [T][H * dim] = exp(-exp_a[h] * softplus(a + dt_bias)).
struct DeltaPrepP {
    float* qkv;
    int64_t ld_qkv;
    float* proj;
    int64_t ld;
    int b_col;
    float* a;
    const float* dt_bias;   // [H * dim]
    const float* exp_a;     // [H]: exp(A_log)
    int H, G, dim, vdim;
};
int delta_prep(const DeltaPrepP& p, int T, hipStream_t st);
// Per entry {first packed row, rows, slot, first position} and head h (key head h / (H / G)), the fp32
// state S [dim][vdim] at state + slot * slot_stride + state_off + h * dim * vdim walks the rows in
// order: S = diag(g) S; u = beta (v - S^T k); S += k u^T; out[t, h] = S^T q.  An entry whose first
// position is 0 (or read_state = 0) starts from S = 0; write_state = 0 leaves the slot's state alone.
struct DeltaScanP {
    const float* qkv;
    int64_t ld_qkv;
    const float* beta;      // beta[t * ld_beta + h]
    int64_t ld_beta;
    const float* g;         // [T][H * dim]
    const int4* entries;
    int n_entries;
    int H, G, dim, vdim;
    float* state;
    int64_t slot_stride, state_off;
    int read_state;         // 0: start from zero; 1: read the state unless the entry starts at position 0; 2: always read
    int write_state;
    float* out;             // [T][H * vdim]
    // pieces of long entries (entries {first packed row, rows, piece index, 0}, state = per-piece end states): with
    // trans [pieces][H][dim][dim] the piece's transition matrix M (s_end = M s_in + s_loc) is written there and
    // w_out [T][H * dim] receives w_t = M_t^T q_t, M_t the transition from the piece's start to row t
    float* trans;
    float* w_out;
};
int delta_scan(const DeltaScanP& p, hipStream_t st);
// Walks every entry's pieces (spans {first piece, pieces, slot, first position}): s_in[c] = the state entering piece
// c, from the slot's state (zero at position 0) through s <- M_c s + s_loc[c]; the slot's state = what leaves the
// last piece (write_state).  s_loc, s_in [pieces][H][dim][vdim].
struct DeltaCarryP {
    const int4* spans;
    int n_spans;
    int H, dim, vdim;
    const float* s_loc;
    const float* trans;
    float* s_in;
    float* state;
    int64_t slot_stride, state_off;
    int write_state;
};
int delta_carry(const DeltaCarryP& p, hipStream_t st);
// out[t, h, :] += s_in[piece of t][h]^T w[t, h, :] over the pieces {first packed row, rows (<= 64), piece index, 0}
struct DeltaApplyP {
    const int4* chunks;
    int n_chunks, max_rows;
    int H, dim, vdim;
    const float* s_in;
    const float* w;
    float* out;
};
int delta_apply(const DeltaApplyP& p, hipStream_t st);
// Rows of W: x = xin + (wb ? rms(v) * (w_one + wb) : v) (when v) + add (when add); then (when wn)
// h = rms(x) * (w_one + wn) with its bf16 image.  xin may be x.  w_one = 1: weight vectors stored
// around zero; 0: plain weights.
// copies > 1: h is written `copies` times, `plane` elements apart (the rows of several residual streams start equal).
int add_norm(float* x, const float* xin, const float* v, const float* wb, const float* add, const float* wn, float* h, uint16_t* h_bf,
             int T, int W, float eps, hipStream_t st, float w_one = 1.0f, int copies = 1, int64_t plane = 0);

// The producers below also write the bf16 image of their result when the *_bf pointer is set
// (bf16 engines: the next product reads it; no separate rounding pass).
// out[t] = E[tok[t]] * scale; with pos (the rows' positions) and freq (double [ceil(W / 2)]) the
// sinusoidal position vector is added: entry 2i = sin(pos * freq[i]), entry 2i + 1 = cos of it
int embed_rows(const void* E, bool w_f32, const int32_t* tok, float* out, uint16_t* out_bf, int T, int W, int vocab,
               hipStream_t st, float scale = 1.0f, const int32_t* pos = nullptr, const double* freq = nullptr);
int head_gate(float* v, uint16_t* v_bf, const float* proj, int64_t ld, int g_col, int heads, int vd, int T, hipStream_t st);
// y = (x ? x : 0) + gain * v / sqrt(mean(v^2) + eps), rows of W
int postnorm_add(const float* x, const float* v, float* y, uint16_t* y_bf, int T, int W, float gain, float eps, hipStream_t st);
// out[i] = gain * rms(x[rows[i]]) (* (w_one + w1p) when w1p)
int final_rows(const float* x, const int32_t* rows, float* out, uint16_t* out_bf, int n, int W, float gain, const float* w1p,
               float eps, hipStream_t st, float w_one = 1.0f);
int depth_mix(const float* stack, int64_t stride, const float* a, int n, float* x, uint16_t* x_bf, int64_t count, hipStream_t st);
// a[m, j] = act(gu[m, j]) * gu[m, ff + j]; act 0: silu, 1: the tanh form of gelu
int silu_mul(const float* gu, float* a, uint16_t* a_bf, int64_t M, int ff, hipStream_t st, int act = 0);
// a = ap u^2 + u / 2 where u > 0, else aq (exp(u) - 1 - u) + u / 2; n elements
int xielu(const float* u, float* a, uint16_t* a_bf, int64_t n, float ap, float aq, hipStream_t st);
// mode 0: score = sigmoid(z) of the `top` largest z = W_r y; mode 1: z = W_r y + bias, score = the
// softmax over the `top` largest z alone.  Ties: the lower index.
int route_topk(const float* y, const void* Wr, const float* bias, bool w_f32, int T, int W, int E, int top, int mode, int32_t* sel,
               float* score, hipStream_t st);
// s = softmax over all E router outputs; chosen by s + corr inside the `keep` best of `groups` equal
// groups of neighbours (a group ranks by its largest s + corr), `top` of them; score = s of the
// chosen / (their sum + 1e-20) * scale.  Ties: the lower index.
int route_grouped(const float* y, const void* Wr, const float* corr, bool w_f32, int T, int W, int E, int top, int groups, int keep,
                  float scale, int32_t* sel, float* score, hipStream_t st);
int moe_group(const int32_t* sel, int n, int E, int32_t* cnt, int32_t* off, int32_t* slot_of, hipStream_t st);
// score (may be null: 1) scales the gathered input rows / the combined output rows
int moe_gather(const float* y, const float* score, const int32_t* slot_of, int T, int top, int W, float* xg, uint16_t* xg_bf,
               hipStream_t st);
// sel / n_real / y: a chosen expert >= n_real is an identity expert whose output is the row's input y
int moe_combine(const float* yd, const int32_t* slot_of, const float* score, int T, int top, int W, float* f, hipStream_t st,
                const int32_t* sel = nullptr, int n_real = 0, const float* y = nullptr);
int argmax_rows(const float* x, int M, int64_t V, int32_t* ids, hipStream_t st);
int rows_to_bf16(const float* x, uint16_t* y, int64_t n, hipStream_t st);
int rows_to_bf16_strided(const float* x, int64_t ldx, uint16_t* y, int64_t ldy, int64_t M, int K, hipStream_t st);
int bf16_to_f32(const uint16_t* x, float* y, int64_t n, hipStream_t st);

}  // namespace lay
}  // namespace qie
