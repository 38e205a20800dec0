// engine_layered.hip — the engine tier for models given as a per-layer program
// (qie_engine_create_layered, qie_engine_put_tensor, qie_batch_step; qie_engine.h).
//
// A layered engine is a qie_engine whose `lm` holds the architecture and the device weights; a
// batch of it is a paged qie_batch whose pool holds, per layer run, the rows its mixer caches
// (latent rows, or K and V rows of a grouped-query attention), whose `lb` holds the step's
// activations and, for recurrent mixers and convolutions over time, one fp32 state per slot and layer run (recurrent
// states, the convolutions' last inputs).  Slots, the block table and the page pool are the
// batch's own (ensure_pages / drop_pages / flush_table, qie_batch_release, qie_batch_page_stats).
//
// A step packs the rows of all entries (portions of prompts and single tokens alike) end to
// end; every projection runs once over all rows, the cache append and the attention address
// their rows through (slot, position) pairs.  fp32: residual stream, norms, router, scores,
// softmax, rotary angles (tables built in double on the host).  compute_f32 = 0 rounds matrix
// operands to bf16 (weights are bf16, the cache rows are stored as bf16); = 1 keeps everything
// fp32.
#include "engine_impl.hpp"
#include "k_layered.hpp"

#include <cmath>
#include <cstring>
#include <map>
#include <string>

namespace qie {

struct HostTensor {
    int dtype = 0;   // 0 bf16 words, 1 int32, 2 fp32
    std::vector<int64_t> shape;
    std::vector<uint8_t> data;
    int64_t numel() const {
        int64_t n = 1;
        for (int64_t s : shape) n *= s;
        return n;
    }
};

struct RopeTab {
    double base;
    int dims;
    qie_rot_scaling sc;   // factor 0: unscaled frequencies
    float* cs;
    float* sn;
};

struct LayerDev {
    qie_layer_desc d{};
    int cache_layer = 0;   // the layer whose cache rows this layer reads
    int rope = 0;
    void* w_in = nullptr;   // [q ; dkv ; g] rows (kv_from layers: [q ; g])
    int n_in = 0, g_col = 0;
    float* dkv_norm = nullptr;
    void* uk_t = nullptr;   // [heads][kv_rank][dim]
    void* uv = nullptr;     // [heads * vdim][kv_rank]
    void* wo = nullptr;     // [width][heads * vdim]
    float g1 = 1.f, g2 = 1.f;
    void* w_gu = nullptr;     // dense [2 ff][width]; moe [experts][2 ff][width]
    void* w_down = nullptr;   // dense [width][ff];   moe [experts][width][ff]
    void* w_router = nullptr;
    float* dwa = nullptr;     // [i + 2]
    // QIE_MIXER_GQA / QIE_MIXER_GQA_RECURRENT: w_in = [q ; k ; (v) ; rec q ; rec f ; rec v] rows,
    // wo = [W_o of the attention | W_o of the recurrence] columns
    int col_k = 0, col_v = -1, col_rq = 0, col_rf = 0, col_rv = 0, n_cat = 0, cat_rec = 0;
    int rope_v = 0;
    float *qn_w = nullptr, *kn_w = nullptr, *r1 = nullptr, *r2 = nullptr;
    float *rec_fb = nullptr, *rec_lower = nullptr, *rec_norm = nullptr;
    // sandwich blocks: weight vectors of the four norms (pre-norm blocks: n1, n2); biased routers
    float *n1 = nullptr, *n1b = nullptr, *n2 = nullptr, *n2b = nullptr;
    float* router_b = nullptr;
    // attention options: head slopes of the linear distance bias, the sigmoid weights' bias per head,
    // the column of the head gates inside the fused projection (-1: none)
    float *slopes = nullptr, *pb = nullptr;
    int col_gate = -1;
    // QIE_MIXER_MINGRU: w_in = [z ; x ; g] rows, wo = W_o; biases of z and x
    float *mg_zb = nullptr, *mg_xb = nullptr;
    // xIELU: softplus(p), 1/2 + softplus(q); the grouped router's correction
    float act_p = 0.f, act_q = 0.f;
    float* correction = nullptr;
    // attention options: bias vectors of q and k, the softmax sink per head
    float *q_bias = nullptr, *k_bias = nullptr, *sink = nullptr;
    // latent queries through a latent of their own: w_in = [dq ; (dkv)] rows (n_pre of them), the
    // latent's norm weight, W_uq [heads * (dim + rot_dim)][q_rank]
    void* w_uq = nullptr;
    float* dq_norm = nullptr;
    int n_pre = 0;
    // hyper-connections of sublayer 1 (mixer) and 2 (feed-forward); the input convolution's taps [width][taps]
    float *hc_in[2] = {nullptr, nullptr}, *hc_out[2] = {nullptr, nullptr}, *hc_mix[2] = {nullptr, nullptr};
    float* canon = nullptr;
    // QIE_MIXER_CHANNEL_DELTA: w_in = [q ; k ; v ; b ; a1 ; g1] rows, W_a2, W_g2, the three short
    // convolutions' taps end to end [2 G dim + H vdim][conv], exp(A_log), dt_bias, the head norm's weight
    void *w_a2 = nullptr, *w_g2 = nullptr;
    float *dl_conv = nullptr, *dl_exp_a = nullptr, *dl_dt_bias = nullptr, *dl_norm = nullptr;
    int col_b = 0, col_a1 = 0, col_g1 = 0, rank_a = 0, rank_g = 0;
};

// One execution of a layer: layers of a repeated group run several times, each run with its
// own cache region and recurrent state.
struct LayerRun {
    int layer = 0;
    bool add_embed = false;   // the embedding rows are added to the stream before this run
};

struct LayeredModel {
    qie_arch_desc a{};
    std::vector<qie_layer_desc> descs;
    bool f32 = false;
    std::map<std::string, HostTensor> host;
    std::vector<LayerDev> L;
    std::vector<RopeTab> ropes;
    void* embed = nullptr;
    void* head = nullptr;
    float g_final = 1.f;
    float* w_final = nullptr;   // sandwich and pre-norm blocks: the output norm's weight vector
    float* w_embed = nullptr;   // the embedding rows' norm (embed_norm)
    double* pos_freq = nullptr; // sinusoidal positions: 10000^(-2i / width), i < ceil(width / 2)
    std::vector<LayerRun> runs;
    bool loops = false;
    std::vector<void*> allocs;
    bool final = false;
    size_t esz() const { return f32 ? 4 : 2; }
};

struct LayeredBatch {
    std::vector<int64_t> layer_off;   // per layer run: element offset of its (K) rows inside a page
    std::vector<int64_t> v_off;       // per layer run: its V rows (grouped-query attention)
    std::vector<int64_t> state_off;   // per layer run: its recurrent state inside a slot's state
    std::vector<int64_t> conv_off;    // per layer run: the last inputs of its short convolutions (delta rule)
    std::vector<int64_t> canon_off;   // per layer run: the last normed mixer inputs (input convolution)
    float *pre = nullptr, *aux = nullptr;   // first-stage projections / convolved q, k, v; second-stage gate logits
    float* dw = nullptr;                    // delta rule in pieces: the rows' transformed queries [rows][heads * dim]
    int64_t m_pre = 0, m_aux = 0, m_dw = 0;
    int32_t* row_k = nullptr;         // a row's index inside its entry
    float* state = nullptr;           // [slots][slot_state] fp32
    int64_t slot_state = 0;
    int4* d_ent = nullptr;            // the step's entries {first packed row, rows, slot, first position}
    int64_t ent_cap = 0;
    int n_ent = 0;
    std::vector<int4> h_ent;
    int4* d_qgroups = nullptr;        // matrix-core grouped-query attention: 16-row groups of the step's entries
    int64_t qgroups_cap = 0;
    int n_qgroups = 0;
    std::vector<int4> h_qgroups;
    // recurrent mixers, long entries: pieces of kScanPiece rows scanned side by side (lay::gated_carry)
    int4 *d_chunks = nullptr, *d_spans = nullptr;
    int64_t chunks_cap = 0;
    int n_chunks = 0, max_count = 0;
    std::vector<int4> h_chunks, h_spans;
    float *s_loc = nullptr, *s_in = nullptr, *s_decay = nullptr;
    int64_t scan_cap = 0;             // pieces the three buffers hold
    int64_t m_state = 0, m_hd = 0;    // largest state / gate row count of a layer run
    // bf16 K / V caches on the matrix-core attention: V rows stored [kv_heads][vdim][page_tokens].  Per layer run
    // (vt_of): a grouped-query mixer whose sizes fit that kernel; v_transposed: any run does.
    bool v_transposed = false;
    std::vector<char> vt_of;
    float *gpart_o = nullptr, *gpart_ml = nullptr;   // its key-split partials
    int64_t gpart_cap = 0;            // (group, tile, split) units they hold
    int64_t cap = 0, want_cap = 0;
    float *stack = nullptr, *x = nullptr, *proj = nullptr, *qabs = nullptr, *olat = nullptr, *ov = nullptr, *mix = nullptr,
          *y = nullptr, *gu = nullptr, *act = nullptr, *ffo = nullptr, *xg = nullptr, *yd = nullptr, *score = nullptr,
          *xn = nullptr, *logits = nullptr, *keep = nullptr;
    uint16_t* logits_bf = nullptr;
    // bf16 engines: images written by the producing kernels (layer input, post-mixer stream, gated
    // head outputs, activations, gathered expert rows, normed output rows)
    uint16_t *x_bf = nullptr, *y_bf = nullptr, *ov_bf = nullptr, *act_bf = nullptr, *xg_bf = nullptr, *xn_bf = nullptr;
    uint16_t* abf = nullptr;      // bf16 image of a product's left operand, where no producer wrote one (bf16 engines: the MFMA / GEMV kernels read bf16)
    int64_t m_abf = 0;            // its elements per row
    // matrix-core attention: row groups per head count, key-split partials
    std::map<int, std::pair<int, int64_t>> groups;   // heads -> (group count, offset into d_groups) of this step
    int4* d_groups = nullptr;
    int64_t groups_cap = 0;
    std::vector<int4> h_groups;
    float *part_o = nullptr, *part_ml = nullptr;
    int64_t part_cap = 0;         // (group, split) units the partials hold
    // the cache pages carry the key-interleaved copy of c: per layer (il_of; a borrowing layer follows the layer
    // whose rows it reads), interleaved: any layer does
    bool interleaved = false;
    std::vector<char> il_of;
    // per-expert products of prompt-sized steps run on side streams beside the engine's (every
    // expert's GEMM alone covers a fraction of the chip); default priority, joined by events
    static constexpr int kSide = 3;
    hipStream_t side[kSide] = {nullptr, nullptr, nullptr};
    hipEvent_t ev_fork = nullptr, ev_join[kSide] = {nullptr, nullptr, nullptr};
    // hipGraphs of small steps (decoding): one per step shape (rows, wanted rows, row groups per head
    // count), captured the second time a shape is seen (the first run makes every allocation);
    // every per-step value is read from device memory, so a replay only needs the uploads before it
    std::map<std::vector<int>, std::pair<int, hipGraphExec_t>> graphs;   // shape -> (times seen, exec or null)
    int64_t graph_replays = 0;
    std::vector<int32_t> h_off;   // host copy of the expert row offsets (prompt-sized steps)
    int32_t *row_slot = nullptr, *row_pos = nullptr, *tok = nullptr, *want = nullptr, *sel = nullptr, *cnt = nullptr,
            *off = nullptr, *slot_of = nullptr, *d_ids = nullptr, *d_step = nullptr;
    int32_t* h_stage = nullptr;   // pinned: row_slot, row_pos, tok of a step
    int64_t h_stage_rows = 0;
    int last_T = 0, last_want = 0;
    int64_t steps = 0;
    bool keep_on = false;
    // per-row maxima over the layers (scratch sizing)
    int64_t m_in = 0, m_hr = 0, m_hv = 0, m_gu = 0, m_act = 0, m_top = 0, m_e = 0, m_r = 0, m_vd = 0;
};

static inline float bf16_to_float(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t float_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static float host_elem(const HostTensor& t, int64_t i) {
    if (t.dtype == 0) return bf16_to_float(((const uint16_t*)t.data.data())[i]);
    if (t.dtype == 2) return ((const float*)t.data.data())[i];
    return (float)((const int32_t*)t.data.data())[i];
}

static int lm_alloc(LayeredModel* m, void** p, size_t bytes) {
    QIE_TRY(dmalloc(p, bytes));
    m->allocs.push_back(*p);
    return 0;
}

static const HostTensor* lm_find(LayeredModel* m, const std::string& name, std::initializer_list<int64_t> shape) {
    auto it = m->host.find(name);
    if (it == m->host.end()) {
        fail(-22, "layered weights: tensor '%s' is missing", name.c_str());
        return nullptr;
    }
    const HostTensor& t = it->second;
    std::vector<int64_t> want(shape);
    if (t.shape != want) {
        std::string got, exp;
        for (int64_t s : t.shape) got += std::to_string(s) + " ";
        for (int64_t s : want) exp += std::to_string(s) + " ";
        fail(-22, "layered weights: tensor '%s' has shape [%s], the architecture needs [%s]", name.c_str(), got.c_str(),
             exp.c_str());
        return nullptr;
    }
    if (t.dtype == 1) {
        fail(-22, "layered weights: tensor '%s' is an integer table", name.c_str());
        return nullptr;
    }
    return &t;
}

// rows [r0, r0 + t.rows) of a device matrix of `cols` columns in the model's weight type
static int lm_upload_rows(LayeredModel* m, void* dev, int64_t r0, int64_t cols, const HostTensor& t,
                          const std::vector<int64_t>* perm = nullptr) {
    const int64_t n = t.numel();
    char* dst = (char*)dev + (size_t)r0 * cols * m->esz();
    if (m->f32) {
        std::vector<float> tmp(n);
        for (int64_t i = 0; i < n; i++) tmp[i] = host_elem(t, perm ? (*perm)[i] : i);
        QIE_HIP(hipMemcpy(dst, tmp.data(), (size_t)n * 4, hipMemcpyHostToDevice));
    } else {
        std::vector<uint16_t> tmp(n);
        for (int64_t i = 0; i < n; i++) {
            const int64_t s = perm ? (*perm)[i] : i;
            tmp[i] = t.dtype == 0 ? ((const uint16_t*)t.data.data())[s] : float_to_bf16(host_elem(t, s));
        }
        QIE_HIP(hipMemcpy(dst, tmp.data(), (size_t)n * 2, hipMemcpyHostToDevice));
    }
    return 0;
}

static int lm_floats(LayeredModel* m, float** dev, const HostTensor& t) {
    const int64_t n = t.numel();
    std::vector<float> tmp(n);
    for (int64_t i = 0; i < n; i++) tmp[i] = host_elem(t, i);
    QIE_TRY(lm_alloc(m, (void**)dev, (size_t)n * 4));
    QIE_HIP(hipMemcpy(*dev, tmp.data(), (size_t)n * 4, hipMemcpyHostToDevice));
    return 0;
}

static int lm_rope(LayeredModel* m, qie_engine* e, double base, int dims, int* index, const qie_rot_scaling* scp = nullptr) {
    qie_rot_scaling sc{};
    if (scp && scp->factor > 0.f) sc = *scp;
    for (size_t i = 0; i < m->ropes.size(); i++)
        if (m->ropes[i].base == base && m->ropes[i].dims == dims && memcmp(&m->ropes[i].sc, &sc, sizeof(sc)) == 0) {
            *index = (int)i;
            return 0;
        }
    const int half = dims / 2, rows = e->opts.max_ctx;
    std::vector<float> cs((size_t)rows * half), sn((size_t)rows * half);
    for (int j = 0; j < half; j++) {
        double f = std::pow(base, -2.0 * j / dims);
        if (sc.factor > 0.f) {   // by wavelength: short ones stay, long ones slow down by the factor, a blend between
            const double lam = 2.0 * M_PI / f, orig = sc.original;
            if (lam > orig / sc.low)
                f = f / sc.factor;
            else if (lam >= orig / sc.high) {
                const double t = (orig / lam - sc.low) / ((double)sc.high - sc.low);
                f = (1.0 - t) * f / sc.factor + t * f;
            }
        }
        for (int p = 0; p < rows; p++) {
            cs[(size_t)p * half + j] = (float)std::cos(p * f);
            sn[(size_t)p * half + j] = (float)std::sin(p * f);
        }
    }
    RopeTab t{base, dims, sc, nullptr, nullptr};
    QIE_TRY(lm_alloc(m, (void**)&t.cs, cs.size() * 4 + 16));
    QIE_TRY(lm_alloc(m, (void**)&t.sn, sn.size() * 4 + 16));
    QIE_HIP(hipMemcpy(t.cs, cs.data(), cs.size() * 4, hipMemcpyHostToDevice));
    QIE_HIP(hipMemcpy(t.sn, sn.data(), sn.size() * 4, hipMemcpyHostToDevice));
    *index = (int)m->ropes.size();
    m->ropes.push_back(t);
    return 0;
}

void layered_engine_destroy(qie_engine* e) {
    if (!e || !e->lm) return;
    for (void* p : e->lm->allocs) hipFree(p);
    delete e->lm;
    e->lm = nullptr;
}

#define LM_GET(var, name, ...)                                   \
    const HostTensor* var = lm_find(m, name, {__VA_ARGS__});     \
    if (!var) return -22

// weight vector of a norm (sandwich blocks), length n
static int lm_vector(LayeredModel* m, float** dev, const std::string& name, int64_t n) {
    const HostTensor* t = lm_find(m, name, {n});
    if (!t) return -22;
    return lm_floats(m, dev, *t);
}

// Fused input rows and output columns of a grouped-query attention, alone ('mix.') or beside a
// gated recurrence ('mix.left.' / 'mix.right.').
static int finalize_gqa_mixer(qie_engine* e, LayeredModel* m, int i) {
    LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    const qie_gqa_desc& a = d.gqa;
    const bool rec = d.mixer == QIE_MIXER_GQA_RECURRENT;
    const int64_t W = m->a.width;
    const std::string pl = "l" + std::to_string(i) + ".", pa = pl + (rec ? "mix.left." : "mix."), pr = pl + "mix.right.";
    const int64_t nq = (int64_t)a.heads * a.dim, nk = (int64_t)a.kv_heads * a.dim, nv = a.values_are_keys ? 0 : (int64_t)a.kv_heads * a.vdim;
    const int64_t rq = rec ? (int64_t)d.rec.heads * d.rec.dim : 0, rv = rec ? (int64_t)d.rec.heads * d.rec.vdim : 0;
    L.col_k = (int)nq;
    L.col_v = a.values_are_keys ? -1 : (int)(nq + nk);
    const int64_t ng = a.out_gate ? (int64_t)a.heads * a.vdim : a.head_gate ? a.heads : 0;
    L.col_gate = ng ? (int)(nq + nk + nv) : -1;
    L.col_rq = (int)(nq + nk + nv + ng);
    L.col_rf = (int)(L.col_rq + rq);
    L.col_rv = (int)(L.col_rf + rq);
    L.n_in = (int)(L.col_rv + rv);
    QIE_TRY(lm_alloc(m, &L.w_in, (size_t)L.n_in * W * m->esz()));
    LM_GET(tq, pa + "q", nq, W);
    LM_GET(tk, pa + "k", nk, W);
    QIE_TRY(lm_upload_rows(m, L.w_in, 0, W, *tq));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_k, W, *tk));
    if (!a.values_are_keys) {
        LM_GET(tv, pa + "v", nv, W);
        QIE_TRY(lm_upload_rows(m, L.w_in, L.col_v, W, *tv));
    }
    if (a.qk_norm == QIE_QKNORM_WEIGHT) {
        QIE_TRY(lm_vector(m, &L.qn_w, pa + "q.norm", a.dim));
        QIE_TRY(lm_vector(m, &L.kn_w, pa + "k.norm", a.dim));
    }
    if (a.dist_bias) {
        QIE_TRY(lm_vector(m, &L.r1, pa + "r1", a.heads));
        QIE_TRY(lm_vector(m, &L.r2, pa + "r2", a.heads));
    }
    if (ng) {
        LM_GET(tg, pa + "g", ng, W);
        QIE_TRY(lm_upload_rows(m, L.w_in, L.col_gate, W, *tg));
    }
    if (a.qk_bias) {
        QIE_TRY(lm_vector(m, &L.q_bias, pa + "q.b", nq));
        QIE_TRY(lm_vector(m, &L.k_bias, pa + "k.b", nk));
    }
    if (a.sink) QIE_TRY(lm_vector(m, &L.sink, pa + "sink", a.heads));
    if (a.weights == QIE_WEIGHTS_SIGMOID) QIE_TRY(lm_vector(m, &L.pb, pa + "pb", a.heads));
    if (a.slope_bias) {
        HostTensor sl;
        sl.dtype = 2;
        sl.shape = {(int64_t)a.heads};
        sl.data.resize((size_t)a.heads * 4);
        for (int h = 0; h < a.heads; h++) ((float*)sl.data.data())[h] = (float)std::exp2(-8.0 * (h + 1) / a.heads);
        QIE_TRY(lm_floats(m, &L.slopes, sl));
    }
    if (a.rot_dims > 0) QIE_TRY(lm_rope(m, e, (double)a.rot_base, a.rot_dims, &L.rope, &a.rot_scaling));
    if (a.rot_values) QIE_TRY(lm_rope(m, e, (double)a.rot_base, a.vdim, &L.rope_v));
    const int64_t ca = (int64_t)a.heads * a.vdim;
    L.cat_rec = (int)ca;
    L.n_cat = (int)(ca + rv);
    QIE_TRY(lm_alloc(m, &L.wo, (size_t)W * L.n_cat * m->esz()));
    LM_GET(to, pa + "o", W, ca);
    if (!rec) {
        QIE_TRY(lm_upload_rows(m, L.wo, 0, ca, *to));
        return 0;
    }
    LM_GET(trq, pr + "q", rq, W);
    LM_GET(trf, pr + "f", rq, W);
    LM_GET(trv, pr + "v", rv, W);
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_rq, W, *trq));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_rf, W, *trf));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_rv, W, *trv));
    QIE_TRY(lm_vector(m, &L.rec_fb, pr + "f.b", rq));
    QIE_TRY(lm_vector(m, &L.rec_lower, pr + "lower", rq));
    QIE_TRY(lm_vector(m, &L.rec_norm, pr + "norm", d.rec.vdim));
    LM_GET(tro, pr + "o", W, rv);
    {   // [W][ca] and [W][rv] side by side: one product over the concatenated head outputs
        HostTensor cat;
        cat.dtype = 2;
        cat.shape = {W, (int64_t)L.n_cat};
        cat.data.resize((size_t)W * L.n_cat * 4);
        float* c = (float*)cat.data.data();
        for (int64_t r = 0; r < W; r++) {
            for (int64_t k = 0; k < ca; k++) c[r * L.n_cat + k] = host_elem(*to, r * ca + k);
            for (int64_t k = 0; k < rv; k++) c[r * L.n_cat + ca + k] = host_elem(*tro, r * rv + k);
        }
        QIE_TRY(lm_upload_rows(m, L.wo, 0, L.n_cat, cat));
    }
    return 0;
}

static int finalize_ff(LayeredModel* m, int i);

// minGRU: fused input rows [z ; x ; g], the two bias vectors, W_o
static int finalize_mingru(LayeredModel* m, int i) {
    LayerDev& L = m->L[i];
    const int64_t W = m->a.width, n = L.d.mingru.width;
    const std::string px = "l" + std::to_string(i) + ".mix.";
    L.n_in = (int)(3 * n);
    L.n_cat = (int)n;
    QIE_TRY(lm_alloc(m, &L.w_in, (size_t)L.n_in * W * m->esz()));
    LM_GET(tz, px + "z", n, W);
    LM_GET(tx, px + "x", n, W);
    LM_GET(tg, px + "g", n, W);
    QIE_TRY(lm_upload_rows(m, L.w_in, 0, W, *tz));
    QIE_TRY(lm_upload_rows(m, L.w_in, n, W, *tx));
    QIE_TRY(lm_upload_rows(m, L.w_in, 2 * n, W, *tg));
    QIE_TRY(lm_vector(m, &L.mg_zb, px + "z.b", n));
    QIE_TRY(lm_vector(m, &L.mg_xb, px + "x.b", n));
    LM_GET(to, px + "o", W, n);
    QIE_TRY(lm_alloc(m, &L.wo, (size_t)W * n * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.wo, 0, n, *to));
    return 0;
}

// Gated delta rule: fused input rows [q ; k ; v ; b ; a1 ; g1], the second-stage matrices, the three
// convolutions' taps end to end, exp(A_log) in double.  rank_a / rank_g 0: the rows of 'a1' / 'g1'.
static int finalize_delta(LayeredModel* m, int i) {
    LayerDev& L = m->L[i];
    const qie_delta_desc& c = L.d.delta;
    const int64_t W = m->a.width, nk = (int64_t)c.kv_heads * c.dim, nv = (int64_t)c.heads * c.vdim, C = 2 * nk + nv;
    const std::string px = "l" + std::to_string(i) + ".mix.";
    auto rows_of = [&](const std::string& name) -> int64_t {
        auto it = m->host.find(name);
        return it != m->host.end() && it->second.shape.size() == 2 ? it->second.shape[0] : 0;
    };
    L.rank_a = c.rank_a > 0 ? c.rank_a : (int)rows_of(px + "a1");
    L.rank_g = c.rank_g > 0 ? c.rank_g : (int)rows_of(px + "g1");
    QIE_REQUIRE(L.rank_a > 0 && L.rank_g > 0, "layered weights: layer %d: tensors '%sa1' / '%sg1' give no rank", i, px.c_str(), px.c_str());
    L.col_k = (int)nk;
    L.col_v = (int)(2 * nk);
    L.col_b = (int)C;
    L.col_a1 = (int)(C + c.heads);
    L.col_g1 = L.col_a1 + L.rank_a;
    L.n_in = L.col_g1 + L.rank_g;
    L.n_cat = (int)nv;
    QIE_TRY(lm_alloc(m, &L.w_in, (size_t)L.n_in * W * m->esz()));
    LM_GET(tq, px + "q", nk, W);
    LM_GET(tk, px + "k", nk, W);
    LM_GET(tv, px + "v", nv, W);
    LM_GET(tb, px + "b", (int64_t)c.heads, W);
    LM_GET(ta1, px + "a1", (int64_t)L.rank_a, W);
    LM_GET(tg1, px + "g1", (int64_t)L.rank_g, W);
    QIE_TRY(lm_upload_rows(m, L.w_in, 0, W, *tq));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_k, W, *tk));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_v, W, *tv));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_b, W, *tb));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_a1, W, *ta1));
    QIE_TRY(lm_upload_rows(m, L.w_in, L.col_g1, W, *tg1));
    LM_GET(ta2, px + "a2", (int64_t)c.heads * c.dim, (int64_t)L.rank_a);
    LM_GET(tg2, px + "g2", nv, (int64_t)L.rank_g);
    QIE_TRY(lm_alloc(m, &L.w_a2, (size_t)ta2->numel() * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.w_a2, 0, L.rank_a, *ta2));
    QIE_TRY(lm_alloc(m, &L.w_g2, (size_t)tg2->numel() * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.w_g2, 0, L.rank_g, *tg2));
    LM_GET(cq, px + "q.conv", nk, (int64_t)c.conv);
    LM_GET(ck, px + "k.conv", nk, (int64_t)c.conv);
    LM_GET(cv, px + "v.conv", nv, (int64_t)c.conv);
    {
        HostTensor cat;
        cat.dtype = 2;
        cat.shape = {C, (int64_t)c.conv};
        cat.data.resize((size_t)C * c.conv * 4);
        float* f = (float*)cat.data.data();
        int64_t o = 0;
        for (const HostTensor* t : {cq, ck, cv})
            for (int64_t k = 0; k < t->numel(); k++) f[o++] = host_elem(*t, k);
        QIE_TRY(lm_floats(m, &L.dl_conv, cat));
    }
    LM_GET(tal, px + "A_log", (int64_t)c.heads);
    {
        HostTensor ea;
        ea.dtype = 2;
        ea.shape = {(int64_t)c.heads};
        ea.data.resize((size_t)c.heads * 4);
        for (int h = 0; h < c.heads; h++) ((float*)ea.data.data())[h] = (float)std::exp((double)host_elem(*tal, h));
        QIE_TRY(lm_floats(m, &L.dl_exp_a, ea));
    }
    QIE_TRY(lm_vector(m, &L.dl_dt_bias, px + "dt_bias", (int64_t)c.heads * c.dim));
    QIE_TRY(lm_vector(m, &L.dl_norm, px + "norm", (int64_t)c.vdim));
    LM_GET(to, px + "o", W, nv);
    QIE_TRY(lm_alloc(m, &L.wo, (size_t)W * nv * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.wo, 0, nv, *to));
    return 0;
}

static int finalize_layer(qie_engine* e, LayeredModel* m, int i) {
    LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    const std::string pl = "l" + std::to_string(i) + ".", px = pl + "mix.";
    if (m->a.streams > 0) {
        const int64_t n = m->a.streams;
        for (int q = 0; q < (d.ff_kind != QIE_FF_NONE ? 2 : 1); q++) {
            const std::string ph = pl + "hc" + std::to_string(q + 1) + ".";
            QIE_TRY(lm_vector(m, &L.hc_in[q], ph + "in", n));
            QIE_TRY(lm_vector(m, &L.hc_out[q], ph + "out", n));
            LM_GET(tm, ph + "mix", n, n);
            QIE_TRY(lm_floats(m, &L.hc_mix[q], *tm));
        }
    }
    if (m->a.canon_taps > 0) {
        LM_GET(tc, pl + "canon1", (int64_t)m->a.width, (int64_t)m->a.canon_taps);
        QIE_TRY(lm_floats(m, &L.canon, *tc));
    }
    if (m->a.block == QIE_BLOCK_SANDWICH) {
        const int64_t Wn = m->a.width;
        QIE_TRY(lm_vector(m, &L.n1, pl + "norm1", Wn));
        QIE_TRY(lm_vector(m, &L.n1b, pl + "norm1b", Wn));
        if (d.ff_kind != QIE_FF_NONE) {
            QIE_TRY(lm_vector(m, &L.n2, pl + "norm2", Wn));
            QIE_TRY(lm_vector(m, &L.n2b, pl + "norm2b", Wn));
        }
    }
    if (m->a.block == QIE_BLOCK_PRENORM) {
        QIE_TRY(lm_vector(m, &L.n1, pl + "norm1", m->a.width));
        if (d.ff_kind != QIE_FF_NONE) QIE_TRY(lm_vector(m, &L.n2, pl + "norm2", m->a.width));
    }
    if (d.mixer == QIE_MIXER_MINGRU) {
        QIE_TRY(finalize_mingru(m, i));
        return finalize_ff(m, i);
    }
    if (d.mixer == QIE_MIXER_CHANNEL_DELTA) {
        QIE_TRY(finalize_delta(m, i));
        return finalize_ff(m, i);
    }
    if (d.mixer != QIE_MIXER_LATENT_ATTENTION) {
        QIE_TRY(finalize_gqa_mixer(e, m, i));
        return finalize_ff(m, i);
    }
    const int64_t W = m->a.width, H = d.heads, hq = d.dim + d.rot_dim, R = d.kv_rank;
    const bool own = d.kv_from < 0;
    const int64_t n_kv = own ? R + d.rot_dim : 0, n_g = d.head_gate ? H : 0;
    if (d.q_rank > 0) {
        // first stage [dq ; (dkv)] -> the latent's norm -> W_uq fills the q heads of the projection row
        QIE_REQUIRE(!d.head_gate, "layer %d: latent queries and the head gate are not wired together", i);
        const int64_t Q = d.q_rank;
        L.n_pre = (int)(Q + n_kv);
        L.n_in = (int)(H * hq);
        L.g_col = -1;
        QIE_TRY(lm_alloc(m, &L.w_in, (size_t)L.n_pre * W * m->esz()));
        LM_GET(tdq, px + "dq", Q, W);
        QIE_TRY(lm_upload_rows(m, L.w_in, 0, W, *tdq));
        QIE_TRY(lm_vector(m, &L.dq_norm, px + "dq.norm", Q));
        LM_GET(tuq, px + "uq", H * hq, Q);
        QIE_TRY(lm_alloc(m, &L.w_uq, (size_t)tuq->numel() * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_uq, 0, Q, *tuq));
        if (own) {
            LM_GET(tk, px + "dkv", R + d.rot_dim, W);
            LM_GET(tn, px + "dkv.norm", R);
            QIE_TRY(lm_upload_rows(m, L.w_in, Q, W, *tk));
            QIE_TRY(lm_floats(m, &L.dkv_norm, *tn));
        }
    } else {
        LM_GET(tq, px + "q", H * hq, W);
        L.n_in = (int)(H * hq + n_kv + n_g);
        L.g_col = n_g ? (int)(H * hq + n_kv) : -1;
        QIE_TRY(lm_alloc(m, &L.w_in, (size_t)L.n_in * W * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_in, 0, W, *tq));
        if (own) {
            LM_GET(tk, px + "dkv", R + d.rot_dim, W);
            LM_GET(tn, px + "dkv.norm", R);
            QIE_TRY(lm_upload_rows(m, L.w_in, H * hq, W, *tk));
            QIE_TRY(lm_floats(m, &L.dkv_norm, *tn));
        }
        if (n_g) {
            LM_GET(tg, px + "g", H, W);
            QIE_TRY(lm_upload_rows(m, L.w_in, L.g_col, W, *tg));
        }
    }
    LM_GET(tuk, px + "uk", H * d.dim, R);
    {   // [heads][dim][R] -> [heads][R][dim]: the absorbed query is q_nope W_uk,h, a product over dim
        std::vector<int64_t> perm((size_t)H * d.dim * R);
        for (int64_t h = 0; h < H; h++)
            for (int64_t r = 0; r < R; r++)
                for (int64_t k = 0; k < d.dim; k++) perm[(h * R + r) * d.dim + k] = (h * d.dim + k) * R + r;
        QIE_TRY(lm_alloc(m, &L.uk_t, perm.size() * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.uk_t, 0, d.dim, *tuk, &perm));
    }
    LM_GET(tuv, px + "uv", H * d.vdim, R);
    QIE_TRY(lm_alloc(m, &L.uv, (size_t)tuv->numel() * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.uv, 0, R, *tuv));
    LM_GET(to, px + "o", W, H * d.vdim);
    QIE_TRY(lm_alloc(m, &L.wo, (size_t)to->numel() * m->esz()));
    QIE_TRY(lm_upload_rows(m, L.wo, 0, H * d.vdim, *to));
    QIE_TRY(lm_rope(m, e, (double)d.rot_base, d.rot_dims, &L.rope, &d.rot_scaling));
    if (m->a.block == QIE_BLOCK_POSTNORM_GAIN) {
        LM_GET(n1, pl + "norm1");
        L.g1 = host_elem(*n1, 0);
        if (d.ff_kind != QIE_FF_NONE) {
            LM_GET(n2, pl + "norm2");
            L.g2 = host_elem(*n2, 0);
        }
    }
    QIE_TRY(finalize_ff(m, i));
    if (m->a.depth_mix) {
        LM_GET(da, pl + "dwa", (int64_t)i + 2);
        QIE_TRY(lm_floats(m, &L.dwa, *da));
    }
    return 0;
}

static int finalize_ff(LayeredModel* m, int i) {
    LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    const int64_t W = m->a.width;
    const std::string pl = "l" + std::to_string(i) + ".";
    const int64_t ff = d.ff;
    if (d.ff_kind == QIE_FF_DENSE && d.ff_act == QIE_ACT_XIELU) {
        LM_GET(wu, pl + "mlp.up", ff, W);
        LM_GET(wd, pl + "mlp.down", W, ff);
        LM_GET(wa, pl + "mlp.act", (int64_t)2);
        QIE_TRY(lm_alloc(m, &L.w_gu, (size_t)ff * W * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_gu, 0, W, *wu));
        QIE_TRY(lm_alloc(m, &L.w_down, (size_t)W * ff * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_down, 0, ff, *wd));
        auto softplus = [](double z) { return std::log1p(std::exp(-std::fabs(z))) + std::max(z, 0.0); };
        L.act_p = (float)softplus((double)host_elem(*wa, 0));
        L.act_q = (float)(0.5 + softplus((double)host_elem(*wa, 1)));
    } else if (d.ff_kind == QIE_FF_DENSE) {
        LM_GET(wg, pl + "mlp.gate", ff, W);
        LM_GET(wu, pl + "mlp.up", ff, W);
        LM_GET(wd, pl + "mlp.down", W, ff);
        QIE_TRY(lm_alloc(m, &L.w_gu, (size_t)2 * ff * W * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_gu, 0, W, *wg));
        QIE_TRY(lm_upload_rows(m, L.w_gu, ff, W, *wu));
        QIE_TRY(lm_alloc(m, &L.w_down, (size_t)W * ff * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_down, 0, ff, *wd));
    } else if (d.ff_kind == QIE_FF_MOE) {
        const int64_t E = d.experts, ER = E + (d.router == QIE_ROUTER_SOFTMAX_ALL ? d.identity : 0);
        LM_GET(wr, pl + "mlp.router", ER, W);
        QIE_TRY(lm_alloc(m, &L.w_router, (size_t)ER * W * m->esz()));
        QIE_TRY(lm_upload_rows(m, L.w_router, 0, W, *wr));
        if (d.router == QIE_ROUTER_SOFTMAX_OUT) QIE_TRY(lm_vector(m, &L.router_b, pl + "mlp.router.b", E));
        if (d.router == QIE_ROUTER_SOFTMAX_ALL) QIE_TRY(lm_vector(m, &L.correction, pl + "mlp.correction", ER));
        QIE_TRY(lm_alloc(m, &L.w_gu, (size_t)E * 2 * ff * W * m->esz()));
        QIE_TRY(lm_alloc(m, &L.w_down, (size_t)E * W * ff * m->esz()));
        for (int64_t x = 0; x < E; x++) {
            const std::string pe = pl + "mlp.e" + std::to_string(x) + ".";
            LM_GET(wg, pe + "gate", ff, W);
            LM_GET(wu, pe + "up", ff, W);
            LM_GET(wd, pe + "down", W, ff);
            QIE_TRY(lm_upload_rows(m, L.w_gu, x * 2 * ff, W, *wg));
            QIE_TRY(lm_upload_rows(m, L.w_gu, x * 2 * ff + ff, W, *wu));
            QIE_TRY(lm_upload_rows(m, L.w_down, x * W, ff, *wd));
        }
    }
    return 0;
}

// ------------------------------------------------------------------ the step
static int lin(const qie_engine* e, const float* A, int64_t lda, const void* Wt, int64_t ldw, float* Y, int64_t ldy, int M, int N,
               int K, int batch = 1, int64_t sA = 0, int64_t sW = 0, int64_t sY = 0, const int32_t* grp = nullptr) {
    lay::LinearP p{A, lda, Wt, ldw, Y, ldy, M, N, K, batch, sA, sW, sY, e->lm->f32 ? 0 : 1, grp, e->lm->f32 ? 0 : 1};
    return lay::linear(p, e->lm->f32, e->stream);
}

static void drop_graphs(LayeredBatch* s);

// Row count from which a step's expert products run per expert on the MFMA kernels (one
// device-to-host copy of the expert offsets per routed layer); below it the grouped kernel runs
// without a host round trip.
constexpr int kMoeSyncRows = 256;

static bool al16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// y[M, N] = A[M, K] W[N, K]^T on the engine's bf16 kernels (MFMA GEMM, GEMV for few rows) when
// the model runs bf16 operands and the shapes fit them (K a multiple of 8, 16-byte aligned
// operands); `abf` receives the bf16 image of A, row stride K.  Else the plain kernel.
static int dense_on(qie_batch* b, uint16_t* abf, bool staged, const float* A, int64_t lda, const void* Wt, float* Y, int64_t ldy,
                    int M, int N, int K, hipStream_t on = nullptr) {
    const qie_engine* e = b->e;
    const hipStream_t st = on ? on : e->stream;
    if (!e->lm->f32 && abf && K % 8 == 0 && al16(Wt) && al16(abf)) {
        if (!staged) QIE_TRY(lay::rows_to_bf16_strided(A, lda, abf, K, M, K, st));
        qie_linear_args a{};
        a.x = abf; a.ldx = K;
        a.w[0] = Wt; a.seg_rows[0] = N;
        a.M = M; a.K = K; a.N = N;
        a.y = Y; a.ldy = ldy;
        a.epilogue = QIE_EPI_F32;
        const int rc = qie_linear(&a, st);
        if (rc != -22) return rc;   // a shape those kernels do not take: the plain kernel below
    }
    lay::LinearP p{A, lda, Wt, K, Y, ldy, M, N, K, 1, 0, 0, 0, e->lm->f32 ? 0 : 1, nullptr, e->lm->f32 ? 0 : 1};
    return lay::linear(p, e->lm->f32, st);
}
// pre: the bf16 image of A (row stride K) when its producer wrote one
static int dense(qie_batch* b, const float* A, int64_t lda, const void* Wt, float* Y, int64_t ldy, int M, int N, int K,
                 const uint16_t* pre = nullptr) {
    if (pre && lda == K) return dense_on(b, const_cast<uint16_t*>(pre), true, A, lda, Wt, Y, ldy, M, N, K);
    return dense_on(b, b->lb->abf, false, A, lda, Wt, Y, ldy, M, N, K);
}

static lay::LatentCache cache_of(const qie_batch* b) {
    return lay::LatentCache{b->kc, b->seq_stride, b->d_table, b->page_tokens, b->max_pages};
}

static int enq_input_proj(qie_batch* b, int i, const float* xin, int T, const uint16_t* xin_bf = nullptr) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    LayeredBatch* s = b->lb;
    return dense(b, xin, m->a.width, L.w_in, s->proj, L.n_in, T, L.n_in, m->a.width, xin_bf);
}

static int enq_latent_post(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    LayeredBatch* s = b->lb;
    lay::LatentPostP p{};
    p.proj = s->proj;
    p.ld = L.n_in;
    p.row_slot = s->row_slot;
    p.row_pos = s->row_pos;
    p.heads = d.heads; p.dim = d.dim; p.rot = d.rot_dim; p.rot_dims = d.rot_dims; p.R = d.kv_rank;
    p.own_kv = d.kv_from < 0;
    p.norm_w = L.dkv_norm;
    p.eps = m->a.norm_eps;
    p.rope_cos = m->ropes[L.rope].cs;
    p.rope_sin = m->ropes[L.rope].sn;
    p.cache = cache_of(b);
    p.layer_off = s->layer_off[L.cache_layer];   // engines with latent layers run every layer once: run == layer
    p.interleaved = s->il_of[L.cache_layer];
    p.rot_layout = d.rot_layout;
    if (d.q_rank > 0 && p.own_kv) {   // the first-stage product holds [latent queries | compressed row | shared key part]
        p.kv = s->pre + d.q_rank;
        p.kv_ld = L.n_pre;
    }
    return lay::latent_post(p, m->f32, T, e->stream);
}

static int enq_absorb(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayerDev& L = e->lm->L[i];
    const qie_layer_desc& d = L.d;
    LayeredBatch* s = b->lb;
    const int hq = d.dim + d.rot_dim;
    const int64_t HR = (int64_t)d.heads * d.kv_rank, HQ = (int64_t)d.heads * hq;
    return lin(e, s->proj, L.n_in, L.uk_t, d.dim, s->qabs, HR, T, d.kv_rank, d.dim, d.heads, hq, (int64_t)d.kv_rank * d.dim,
               d.kv_rank);
}

static int enq_attention(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    LayeredBatch* s = b->lb;
    lay::LatentAttnP p{};
    p.q_abs = s->qabs;
    p.proj = s->proj;
    p.ld = L.n_in;
    p.row_slot = s->row_slot;
    p.row_pos = s->row_pos;
    const int window = d.window > 0 ? d.window : b->max_ctx;   // 0: every earlier position
    p.heads = d.heads; p.dim = d.dim; p.rot = d.rot_dim; p.R = d.kv_rank; p.window = window;
    p.scale = d.scale;
    p.cache = cache_of(b);
    p.layer_off = s->layer_off[L.cache_layer];
    p.out = s->olat;
    auto it = s->groups.find(d.heads);
    if (s->il_of[L.cache_layer] && it != s->groups.end() && lay::latent_attention_mfma_fits(d.kv_rank, d.rot_dim)) {
        // bf16 cache rows: the matrix-core kernel; enough key splits to fill the chip when the
        // step has few rows (decoding)
        const int ng = it->second.first;
        int S = 1024 * lay::kLatentQG / ng;
        const int nb = window / 32 + 2;
        S = std::max(1, std::min({S, nb, 64}));
        if ((int64_t)ng * S > s->part_cap) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            QIE_REQUIRE(hipStreamIsCapturing(e->stream, &cs) == hipSuccess && cs == hipStreamCaptureStatusNone,
                        "latent attention: scratch growth inside a capture");
            QIE_HIP(hipStreamSynchronize(e->stream));
            drop_graphs(s);
            if (s->part_o) hipFree(s->part_o);
            if (s->part_ml) hipFree(s->part_ml);
            s->part_o = s->part_ml = nullptr;
            s->part_cap = 0;
            const int64_t units = ((int64_t)ng * S + 255) / 256 * 256;
            QIE_TRY(dmalloc((void**)&s->part_o, (size_t)units * 16 * s->m_r * 4));
            QIE_TRY(dmalloc((void**)&s->part_ml, (size_t)units * 16 * 2 * 4));
            s->part_cap = units;
        }
        lay::LatentAttnMfmaP q{};
        q.q_abs = s->qabs; q.proj = s->proj; q.ld = L.n_in;
        q.row_slot = s->row_slot; q.row_pos = s->row_pos;
        q.groups = s->d_groups + it->second.second;
        q.n_groups = ng; q.S = S;
        q.heads = d.heads; q.dim = d.dim; q.rot = d.rot_dim; q.R = d.kv_rank; q.window = window;
        q.scale = d.scale;
        q.cache = p.cache; q.layer_off = p.layer_off;
        q.part_o = s->part_o; q.part_ml = s->part_ml; q.out = s->olat;
        return lay::latent_attention_mfma(q, e->stream);
    }
    return lay::latent_attention(p, m->f32, T, e->stream);
}

// Row groups of a step for the matrix-core attention, one list per distinct head count: heads
// >= 16 split a token's heads into groups of 16; fewer heads put 16 / heads consecutive tokens of
// one entry into a group.
static int build_groups(qie_batch* b, int n_entries, const int32_t* counts) {
    LayeredBatch* s = b->lb;
    const LayeredModel* m = b->e->lm;
    s->groups.clear();
    s->h_groups.clear();
    if (!s->interleaved) return 0;
    const int pad = lay::kLatentQG;
    for (const LayerDev& L : m->L) {
        const int H = L.d.heads;
        if (L.d.mixer != QIE_MIXER_LATENT_ATTENTION || !s->il_of[L.cache_layer] || s->groups.count(H)) continue;
        const int64_t first = (int64_t)s->h_groups.size();
        int row = 0;
        for (int i = 0; i < n_entries; i++) {
            if (H >= 16) {
                for (int k = 0; k < counts[i]; k++)
                    for (int h0 = 0; h0 < H; h0 += 16) s->h_groups.push_back(int4{row + k, 1, h0, std::min(16, H - h0)});
            } else {
                const int tpg = 16 / H;
                for (int k = 0; k < counts[i]; k += tpg) s->h_groups.push_back(int4{row + k, std::min(tpg, counts[i] - k), 0, H});
            }
            // whole units per entry: a unit's groups share the slot
            while ((s->h_groups.size() - first) % pad) s->h_groups.push_back(int4{row, 0, 0, 1});
            row += counts[i];
        }
        s->groups[H] = {(int)(s->h_groups.size() - first), first};
    }
    if ((int64_t)s->h_groups.size() > s->groups_cap) {
        QIE_HIP(hipStreamSynchronize(b->e->stream));
        drop_graphs(s);
        if (s->d_groups) hipFree(s->d_groups);
        s->d_groups = nullptr;
        s->groups_cap = 0;
        const int64_t cap = ((int64_t)s->h_groups.size() + 1023) / 1024 * 1024;
        QIE_TRY(dmalloc((void**)&s->d_groups, (size_t)cap * sizeof(int4)));
        s->groups_cap = cap;
    }
    QIE_HIP(hipMemcpyAsync(s->d_groups, s->h_groups.data(), s->h_groups.size() * sizeof(int4), hipMemcpyHostToDevice,
                           b->e->stream));
    return 0;
}

static int enq_mixer_out(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    LayeredBatch* s = b->lb;
    const int64_t HV = (int64_t)d.heads * d.vdim;
    const int64_t HR = (int64_t)d.heads * d.kv_rank;
    QIE_TRY(lin(e, s->olat, HR, L.uv, d.kv_rank, s->ov, HV, T, d.vdim, d.kv_rank, d.heads, d.kv_rank, (int64_t)d.vdim * d.kv_rank,
                d.vdim));
    if (L.g_col < 0) return dense(b, s->ov, HV, L.wo, s->mix, m->a.width, T, m->a.width, (int)HV);
    QIE_TRY(lay::head_gate(s->ov, s->ov_bf, s->proj, L.n_in, L.g_col, d.heads, d.vdim, T, e->stream));
    return dense(b, s->ov, HV, L.wo, s->mix, m->a.width, T, m->a.width, (int)HV, s->ov_bf);
}

// feed-forward of layer i on rows y -> ffo
static int enq_ff(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    const qie_layer_desc& d = L.d;
    LayeredBatch* s = b->lb;
    const int W = m->a.width, ff = d.ff;
    hipStream_t st = e->stream;
    if (d.ff_kind == QIE_FF_DENSE && d.ff_act == QIE_ACT_XIELU) {
        QIE_TRY(dense(b, s->y, W, L.w_gu, s->gu, ff, T, ff, W, s->y_bf));
        QIE_TRY(lay::xielu(s->gu, s->act, s->act_bf, (int64_t)T * ff, L.act_p, L.act_q, st));
        return dense(b, s->act, ff, L.w_down, s->ffo, W, T, W, ff, s->act_bf);
    }
    if (d.ff_kind == QIE_FF_DENSE) {
        QIE_TRY(dense(b, s->y, W, L.w_gu, s->gu, 2 * ff, T, 2 * ff, W, s->y_bf));
        QIE_TRY(lay::silu_mul(s->gu, s->act, s->act_bf, T, ff, st, d.ff_act == QIE_ACT_GELU_TANH_GATED ? 1 : 0));
        return dense(b, s->act, ff, L.w_down, s->ffo, W, T, W, ff, s->act_bf);
    }
    const int E = d.experts, top = d.top, n = T * top;
    const bool out_w = d.router != QIE_ROUTER_SIGMOID_IN;   // the scores weight the outputs, not the inputs
    const float* in_score = out_w ? nullptr : s->score;
    const float* out_score = out_w ? s->score : nullptr;
    // identity experts follow the real ones in the router's outputs: they get groups of their own in
    // the row order below, no products, and the combine takes the rows' input for them
    const int ER = E + (d.router == QIE_ROUTER_SOFTMAX_ALL ? d.identity : 0);
    const int32_t* id_sel = ER > E ? s->sel : nullptr;
    if (d.router == QIE_ROUTER_SOFTMAX_ALL)
        QIE_TRY(lay::route_grouped(s->y, L.w_router, L.correction, m->f32, T, W, ER, top, d.groups, d.groups_keep, d.route_scale,
                                   s->sel, s->score, st));
    else
        QIE_TRY(lay::route_topk(s->y, L.w_router, L.router_b, m->f32, T, W, E, top, out_w ? 1 : 0, s->sel, s->score, st));
    QIE_TRY(lay::moe_group(s->sel, n, ER, s->cnt, s->off, s->slot_of, st));
    const bool per_expert = !m->f32 && n >= kMoeSyncRows && W % 8 == 0 && ff % 8 == 0;
    QIE_TRY(lay::moe_gather(s->y, in_score, s->slot_of, T, top, W, s->xg, per_expert ? s->xg_bf : nullptr, st));
    if (per_expert) {
        // prompt-sized steps: the expert row ranges come to the host and every expert's rows go
        // through the MFMA kernels; the products are the grouped kernel's, in another order
        s->h_off.resize(E + 1);
        QIE_HIP(hipMemcpyAsync(s->h_off.data(), s->off, (size_t)(E + 1) * 4, hipMemcpyDeviceToHost, st));
        QIE_HIP(hipStreamSynchronize(st));
        // experts round-robin over the engine's stream and the side streams, forked and joined
        // by events around each of the two product phases
        auto fork = [&]() -> int {
            QIE_HIP(hipEventRecord(s->ev_fork, st));
            for (int i = 0; i < LayeredBatch::kSide; i++) QIE_HIP(hipStreamWaitEvent(s->side[i], s->ev_fork, 0));
            return 0;
        };
        auto join = [&]() -> int {
            for (int i = 0; i < LayeredBatch::kSide; i++) {
                QIE_HIP(hipEventRecord(s->ev_join[i], s->side[i]));
                QIE_HIP(hipStreamWaitEvent(st, s->ev_join[i], 0));
            }
            return 0;
        };
        auto lane_of = [&](int x) { return x % (LayeredBatch::kSide + 1) == 0 ? st : s->side[x % (LayeredBatch::kSide + 1) - 1]; };
        QIE_TRY(fork());
        for (int x = 0; x < E; x++) {
            const int r0 = s->h_off[x], cnt = s->h_off[x + 1] - r0;
            if (cnt > 0)
                QIE_TRY(dense_on(b, s->xg_bf + (int64_t)r0 * W, true, s->xg + (int64_t)r0 * W, W,
                                 (const uint16_t*)L.w_gu + (int64_t)x * 2 * ff * W, s->gu + (int64_t)r0 * 2 * ff, 2 * ff, cnt,
                                 2 * ff, W, lane_of(x)));
        }
        QIE_TRY(join());
        QIE_TRY(lay::silu_mul(s->gu, s->act, s->act_bf, n, ff, st));
        QIE_TRY(fork());
        for (int x = 0; x < E; x++) {
            const int r0 = s->h_off[x], cnt = s->h_off[x + 1] - r0;
            if (cnt > 0)
                QIE_TRY(dense_on(b, s->act_bf + (int64_t)r0 * ff, true, s->act + (int64_t)r0 * ff, ff,
                                 (const uint16_t*)L.w_down + (int64_t)x * W * ff, s->yd + (int64_t)r0 * W, W, cnt, W, ff,
                                 lane_of(x)));
        }
        QIE_TRY(join());
        return lay::moe_combine(s->yd, s->slot_of, out_score, T, top, W, s->ffo, st, id_sel, E, s->y);
    }
    QIE_TRY(lin(e, s->xg, W, L.w_gu, W, s->gu, 2 * ff, n, 2 * ff, W, E, 0, (int64_t)2 * ff * W, 0, s->off));
    QIE_TRY(lay::silu_mul(s->gu, s->act, nullptr, n, ff, st));
    QIE_TRY(lin(e, s->act, ff, L.w_down, ff, s->yd, W, n, W, ff, E, 0, (int64_t)W * ff, 0, s->off));
    return lay::moe_combine(s->yd, s->slot_of, out_score, T, top, W, s->ffo, st, id_sel, E, s->y);
}

// ---- grouped-query attention (+ gated recurrence) of layer run r; the branch input is s->y
static lay::GqaAttnP gqa_attn_params(qie_batch* b, int r) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    const qie_gqa_desc& a = L.d.gqa;
    LayeredBatch* s = b->lb;
    lay::GqaAttnP p{};
    p.proj = s->proj; p.ld = L.n_in; p.q_col = 0;
    p.row_slot = s->row_slot; p.row_pos = s->row_pos;
    p.heads = a.heads; p.kv_heads = a.kv_heads; p.dim = a.dim; p.vdim = a.vdim;
    p.mask = a.mask; p.mask_size = a.mask_size; p.scale = a.scale;
    p.r1 = a.dist_bias ? L.r1 : nullptr;
    p.r2 = a.dist_bias ? L.r2 : nullptr;
    p.rot_values = a.rot_values; p.rot_layout = a.rot_layout;
    if (a.rot_values) {
        p.vrope_cos = m->ropes[L.rope_v].cs;
        p.vrope_sin = m->ropes[L.rope_v].sn;
    }
    p.cache = cache_of(b);
    p.k_off = s->layer_off[r];
    p.v_off = s->v_off[r];
    p.v_transposed = s->vt_of[r];
    p.out_scale = L.d.mixer == QIE_MIXER_GQA_RECURRENT ? L.d.gqa_scale : 1.0f;
    p.out = s->ov; p.out_bf = s->ov_bf; p.ld_out = L.n_cat; p.out_col = 0;
    p.slopes = a.slope_bias ? L.slopes : nullptr;
    p.pb = a.weights == QIE_WEIGHTS_SIGMOID ? L.pb : nullptr;
    p.gate_col = (a.head_gate || a.out_gate) ? L.col_gate : -1;
    p.gate_elem = a.out_gate ? 1 : 0;
    p.sink = a.sink ? L.sink : nullptr;
    return p;
}

static int enq_gqa_proj(qie_batch* b, int r, int T) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    return dense(b, s->y, m->a.width, L.w_in, s->proj, L.n_in, T, L.n_in, m->a.width, s->y_bf);
}

static int enq_gqa_post(qie_batch* b, int r, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    const qie_gqa_desc& a = L.d.gqa;
    LayeredBatch* s = b->lb;
    lay::GqaPostP p{};
    p.proj = s->proj; p.ld = L.n_in; p.q_col = 0; p.k_col = L.col_k; p.v_col = L.col_v;
    p.row_slot = s->row_slot; p.row_pos = s->row_pos;
    p.heads = a.heads; p.kv_heads = a.kv_heads; p.dim = a.dim; p.vdim = a.vdim;
    p.qk_norm = a.qk_norm; p.qn_w = L.qn_w; p.kn_w = L.kn_w; p.eps = m->a.norm_eps;
    p.rot_dims = a.rot_dims; p.rot_layout = a.rot_layout;
    if (a.rot_dims > 0) {
        p.rope_cos = m->ropes[L.rope].cs;
        p.rope_sin = m->ropes[L.rope].sn;
    }
    p.rot_values = a.rot_values;
    if (a.rot_values) {
        p.vrope_cos = m->ropes[L.rope_v].cs;
        p.vrope_sin = m->ropes[L.rope_v].sn;
    }
    p.cache = cache_of(b);
    p.k_off = s->layer_off[r];
    p.v_off = s->v_off[r];
    p.v_transposed = s->vt_of[r];
    p.q_temp_every = a.q_temp_every;
    p.q_temp_coef = a.q_temp_coef;
    p.q_bias = a.qk_bias ? L.q_bias : nullptr;
    p.k_bias = a.qk_bias ? L.k_bias : nullptr;
    return lay::gqa_post(p, m->f32, T, e->stream);
}

static int enq_gqa_attention(qie_batch* b, int r, int T) {
    const qie_engine* e = b->e;
    LayeredBatch* s = b->lb;
    const lay::GqaAttnP p = gqa_attn_params(b, r);
    if (p.v_transposed && s->n_qgroups > 0) {
        // enough key splits to fill the chip when the step has few rows (decoding)
        const int tiles = (p.heads + 3) / 4 * 4;
        const int64_t waves = (int64_t)s->n_qgroups * p.heads;
        const int max_blocks = (p.mask == QIE_MASK_CAUSAL ? b->max_ctx : std::min(b->max_ctx, p.mask_size)) / 32 + 2;
        // (a wave walks its key blocks one after the other, each a trip to memory: prompts of a
        // few thousand rows leave too few waves to hide them, so their keys are split as well)
        static const int split_waves = dev_env("QIE_GQA_SPLIT_WAVES", 6144);   // dev A/B knob: waves a launch aims for
        const int S = (int)std::max<int64_t>(1, std::min<int64_t>({split_waves / waves, max_blocks / 4, 32}));
        const int64_t units = (int64_t)s->n_qgroups * tiles * S;
        if (S > 1 && units > s->gpart_cap) {
            hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
            QIE_REQUIRE(hipStreamIsCapturing(e->stream, &cs) == hipSuccess && cs == hipStreamCaptureStatusNone,
                        "gqa attention: scratch growth inside a capture");
            QIE_HIP(hipStreamSynchronize(e->stream));
            drop_graphs(s);
            if (s->gpart_o) hipFree(s->gpart_o);
            if (s->gpart_ml) hipFree(s->gpart_ml);
            s->gpart_o = s->gpart_ml = nullptr;
            s->gpart_cap = 0;
            const int64_t cap = (units + 255) / 256 * 256;
            QIE_TRY(dmalloc((void**)&s->gpart_o, (size_t)cap * 16 * s->m_vd * 4));
            QIE_TRY(dmalloc((void**)&s->gpart_ml, (size_t)cap * 16 * 2 * 4));
            s->gpart_cap = cap;
        }
        lay::GqaAttnMfmaP q{p, s->d_qgroups, s->n_qgroups, S, s->gpart_o, s->gpart_ml, (p.heads / p.kv_heads) % 4 != 0 ? 1 : 0};
        return lay::gqa_attention_mfma(q, e->stream);
    }
    return lay::gqa_attention(p, e->lm->f32, T, e->stream);
}

// Rows of an entry above which the recurrence runs in pieces; rows per piece.
constexpr int kScanLong = 128, kScanPiece = 64;

static int enq_recurrence(qie_batch* b, int r, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    const qie_recurrent_desc& c = L.d.rec;
    LayeredBatch* s = b->lb;
    lay::GatedScanP p{};
    p.proj = s->proj; p.ld = L.n_in; p.q_col = L.col_rq; p.f_col = L.col_rf; p.v_col = L.col_rv;
    p.entries = s->d_ent; p.n_entries = s->n_ent;
    p.heads = c.heads; p.dim = c.dim; p.vdim = c.vdim;
    p.f_bias = L.rec_fb; p.lower = L.rec_lower;
    p.state = s->state; p.slot_stride = s->slot_state; p.state_off = s->state_off[r];
    p.out = s->olat;
    if (s->max_count > kScanLong && s->s_loc) {
        const int64_t n = (int64_t)c.heads * c.dim * c.vdim;
        lay::GatedScanP a = p;       // pieces from zero states: local outputs, end states, gate products
        a.entries = s->d_chunks; a.n_entries = s->n_chunks;
        a.state = s->s_loc; a.slot_stride = n; a.state_off = 0;
        a.decay = s->s_decay;
        QIE_TRY(lay::gated_scan(a, e->stream));
        lay::GatedCarryP k{s->d_spans, s->n_ent, c.heads, c.dim, c.vdim, s->s_loc, s->s_decay, s->s_in, s->state, s->slot_state,
                           s->state_off[r]};
        QIE_TRY(lay::gated_carry(k, e->stream));
        a.state = s->s_in;           // the incoming states' share of every row, summed in the head norm
        a.mode = 1;
        a.decay = nullptr;
        a.out = s->qabs;
        QIE_TRY(lay::gated_scan(a, e->stream));
        return lay::head_norm_rows(s->olat, s->qabs, L.rec_norm, m->a.norm_eps, L.d.rec_scale, c.heads, c.vdim, T, s->ov, s->ov_bf,
                                   L.n_cat, L.cat_rec, e->stream);
    }
    QIE_TRY(lay::gated_scan(p, e->stream));
    return lay::head_norm_rows(s->olat, nullptr, L.rec_norm, m->a.norm_eps, L.d.rec_scale, c.heads, c.vdim, T, s->ov, s->ov_bf, L.n_cat,
                               L.cat_rec, e->stream);
}

static int enq_gqa_mixer(qie_batch* b, int r, int T) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    QIE_TRY(enq_gqa_proj(b, r, T));
    QIE_TRY(enq_gqa_post(b, r, T));
    QIE_TRY(enq_gqa_attention(b, r, T));
    if (L.d.mixer == QIE_MIXER_GQA_RECURRENT) QIE_TRY(enq_recurrence(b, r, T));
    return dense(b, s->ov, L.n_cat, L.wo, s->mix, m->a.width, T, m->a.width, L.n_cat, s->ov_bf);
}

// minGRU of layer run r: the scan over the fused projection rows -> s->ov (gated, with its bf16 image).
// Entries above kScanLong rows run in pieces: piece-local end states and decay products from zero
// states, a carry pass over each entry's pieces, then the pieces again from the states that enter
// them (the same recurrence, regrouped: S_end = decay * S_in + S_local).
static int enq_mingru(qie_batch* b, int r, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    const int n = L.d.mingru.width;
    lay::MinGruScanP p{};
    p.proj = s->proj; p.ld = L.n_in; p.z_col = 0; p.x_col = n; p.g_col = 2 * n;
    p.z_b = L.mg_zb; p.x_b = L.mg_xb;
    p.n = n;
    p.out = s->ov; p.out_bf = s->ov_bf; p.ld_out = n;
    if (s->max_count > kScanLong && s->s_loc) {
        lay::MinGruScanP a = p;
        a.entries = s->d_chunks; a.n_entries = s->n_chunks;
        a.out = nullptr; a.out_bf = nullptr;
        a.end = s->s_loc; a.decay = s->s_decay; a.end_stride = n; a.end_off = 0;
        QIE_TRY(lay::mingru_scan(a, e->stream));
        lay::MinGruCarryP k{s->d_spans, s->n_ent, n, s->s_loc, s->s_decay, s->s_in, s->state, s->slot_state, s->state_off[r]};
        QIE_TRY(lay::mingru_carry(k, e->stream));
        a = p;
        a.entries = s->d_chunks; a.n_entries = s->n_chunks;
        a.init = s->s_in; a.init_stride = n; a.init_off = 0; a.init_if_pos = 0;
        return lay::mingru_scan(a, e->stream);
    }
    p.entries = s->d_ent; p.n_entries = s->n_ent;
    p.init = s->state; p.init_stride = s->slot_state; p.init_off = s->state_off[r]; p.init_if_pos = 1;
    p.end = s->state; p.end_stride = s->slot_state; p.end_off = s->state_off[r];
    return lay::mingru_scan(p, e->stream);
}

static int enq_mingru_mixer(qie_batch* b, int r, int T) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    QIE_TRY(dense(b, s->y, m->a.width, L.w_in, s->proj, L.n_in, T, L.n_in, m->a.width, s->y_bf));
    QIE_TRY(enq_mingru(b, r, T));
    return dense(b, s->ov, L.n_cat, L.wo, s->mix, m->a.width, T, m->a.width, L.n_cat, s->ov_bf);
}

// Latent attention of layer run r on the branch input s->y -> s->mix (pre-norm blocks).
static int enq_latent_proj(qie_batch* b, int i, int T) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    LayeredBatch* s = b->lb;
    const int W = m->a.width;
    if (L.d.q_rank <= 0) return dense(b, s->y, W, L.w_in, s->proj, L.n_in, T, L.n_in, W, s->y_bf);
    // [latent queries | compressed row | shared key part] -> the latent's norm in place -> W_uq
    QIE_TRY(dense(b, s->y, W, L.w_in, s->pre, L.n_pre, T, L.n_pre, W, s->y_bf));
    QIE_TRY(lay::rms_rows(s->pre, L.n_pre, 0, L.d.q_rank, L.dq_norm, 0.f, m->a.norm_eps, s->pre, L.n_pre, nullptr, T, e->stream));
    return dense(b, s->pre, L.n_pre, L.w_uq, s->proj, L.n_in, T, L.n_in, L.d.q_rank);
}

static int enq_latent_mixer(qie_batch* b, int r, int T) {
    const int i = b->e->lm->runs[r].layer;
    QIE_TRY(enq_latent_proj(b, i, T));
    QIE_TRY(enq_latent_post(b, i, T));
    QIE_TRY(enq_absorb(b, i, T));
    QIE_TRY(enq_attention(b, i, T));
    return enq_mixer_out(b, i, T);
}

// Gated delta rule of layer run r: fused projection [q ; k ; v ; b ; a1 ; g1] and the second-stage
// products, then (enq_delta_scan) the short convolutions with silu, the gates, the scan and the gated head norm.
static int enq_delta_proj(qie_batch* b, int r, int T) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    const qie_delta_desc& c = L.d.delta;
    LayeredBatch* s = b->lb;
    const int W = m->a.width;
    QIE_TRY(dense(b, s->y, W, L.w_in, s->proj, L.n_in, T, L.n_in, W, s->y_bf));
    QIE_TRY(dense(b, s->proj + L.col_a1, L.n_in, L.w_a2, s->qabs, (int64_t)c.heads * c.dim, T, c.heads * c.dim, L.rank_a));
    return dense(b, s->proj + L.col_g1, L.n_in, L.w_g2, s->aux, (int64_t)c.heads * c.vdim, T, c.heads * c.vdim, L.rank_g);
}

static int enq_delta_scan(qie_batch* b, int r, int T, bool advance) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    const qie_delta_desc& c = L.d.delta;
    LayeredBatch* s = b->lb;
    const int C = 2 * c.kv_heads * c.dim + c.heads * c.vdim;
    lay::CausalConvP cv{};
    cv.in = s->proj; cv.ld_in = L.n_in; cv.col = 0; cv.C = C; cv.taps = c.conv; cv.w = L.dl_conv;
    cv.row_slot = s->row_slot; cv.row_pos = s->row_pos; cv.row_k = s->row_k;
    cv.state = s->state; cv.slot_stride = s->slot_state; cv.state_off = s->conv_off[r];
    cv.residual = 0; cv.silu = 1;
    cv.out = s->pre; cv.ld_out = C; cv.out_bf = nullptr;
    cv.entries = s->d_ent; cv.n_entries = s->n_ent;
    if (advance)
        QIE_TRY(lay::causal_conv_advance(cv, T, e->stream));
    else
        QIE_TRY(lay::causal_conv(cv, T, e->stream));
    lay::DeltaPrepP pp{s->pre, C, s->proj, L.n_in, L.col_b, s->qabs, L.dl_dt_bias, L.dl_exp_a, c.heads, c.kv_heads, c.dim, c.vdim};
    QIE_TRY(lay::delta_prep(pp, T, e->stream));
    lay::DeltaScanP sp{};
    sp.qkv = s->pre; sp.ld_qkv = C; sp.beta = s->proj + L.col_b; sp.ld_beta = L.n_in; sp.g = s->qabs;
    sp.entries = s->d_ent; sp.n_entries = s->n_ent;
    sp.H = c.heads; sp.G = c.kv_heads; sp.dim = c.dim; sp.vdim = c.vdim;
    sp.state = s->state; sp.slot_stride = s->slot_state; sp.state_off = s->state_off[r];
    sp.read_state = 1; sp.write_state = advance ? 1 : 0;
    sp.out = s->olat;
    if (s->max_count > kScanLong && s->s_loc && s->dw) {
        // long entries: pieces from zero states side by side (end states, transition matrices, transformed
        // queries), a carry over each entry's pieces, then the incoming states' share of every row
        const int64_t n = (int64_t)c.heads * c.dim * c.vdim;
        lay::DeltaScanP a = sp;
        a.entries = s->d_chunks; a.n_entries = s->n_chunks;
        a.state = s->s_loc; a.slot_stride = n; a.state_off = 0;
        a.read_state = 0; a.write_state = 1;
        a.trans = s->s_decay; a.w_out = s->dw;
        QIE_TRY(lay::delta_scan(a, e->stream));
        lay::DeltaCarryP k{s->d_spans, s->n_ent, c.heads, c.dim, c.vdim, s->s_loc, s->s_decay, s->s_in, s->state, s->slot_state,
                           s->state_off[r], advance ? 1 : 0};
        QIE_TRY(lay::delta_carry(k, e->stream));
        lay::DeltaApplyP ap{s->d_chunks, s->n_chunks, kScanPiece, c.heads, c.dim, c.vdim, s->s_in, s->dw, s->olat};
        QIE_TRY(lay::delta_apply(ap, e->stream));
    } else {
        QIE_TRY(lay::delta_scan(sp, e->stream));
    }
    return lay::head_norm_rows(s->olat, nullptr, L.dl_norm, m->a.norm_eps, 1.0f, c.heads, c.vdim, T, s->ov, s->ov_bf, L.n_cat, 0,
                               e->stream, s->aux);
}

static int enq_delta_mixer(qie_batch* b, int r, int T) {
    const LayeredModel* m = b->e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    QIE_TRY(enq_delta_proj(b, r, T));
    QIE_TRY(enq_delta_scan(b, r, T, true));
    return dense(b, s->ov, L.n_cat, L.wo, s->mix, m->a.width, T, m->a.width, L.n_cat, s->ov_bf);
}

// Pre-norm blocks: x += mixer(N1(x)); x += ff(N2(x)) with weights norm_offset + w.  One residual row
// (streams 0): the stream lives in plane 1 of the stack and every residual add is fused with the norm
// that reads its result.  Several rows (hyper-connections): planes 0 .. streams - 1; the update after
// a sublayer, the read-out for the next one and its norm are one kernel.  Either way the last kernel
// of a run makes the next run's input.  With an input convolution the mixer's normed input goes to
// s->x first and h + conv(h) to s->y.
static int enq_run_prenorm(qie_batch* b, int r, int T, bool h_ready, bool* next_ready) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    const int W = m->a.width, n = m->a.streams;
    hipStream_t st = e->stream;
    const int64_t plane = s->cap * W;
    float* x = n > 0 ? s->stack : s->stack + plane;
    const float eps = m->a.norm_eps, w_one = m->a.norm_offset;
    const bool canon = m->a.canon_taps > 0;
    // y: the sublayer result that updates the rows with the coefficients of sublayer q of this layer (null:
    // none); then the read-out with in_next (hyper-connections) normed with wn -> h (null wn: no read-out)
    auto step = [&](const float* y, int q, const float* in_next, const float* wn, bool to_mixer, float* sum) -> int {
        float* h = to_mixer && canon ? s->x : s->y;
        uint16_t* h_bf = to_mixer && canon ? nullptr : s->y_bf;
        if (n > 0) {
            lay::StreamStepP p{x, plane, n, y, y ? L.hc_mix[q] : nullptr, y ? L.hc_out[q] : nullptr, wn ? in_next : nullptr, wn, w_one, eps,
                               h, h_bf, sum, T, W};
            return lay::stream_step(p, st);
        }
        return lay::add_norm(x, x, y, nullptr, nullptr, wn, h, h_bf, T, W, eps, st, w_one);
    };
    if (!h_ready) QIE_TRY(step(nullptr, 0, L.hc_in[0], L.n1, true, nullptr));
    if (canon) {
        lay::CausalConvP cv{};
        cv.in = s->x; cv.ld_in = W; cv.col = 0; cv.C = W; cv.taps = m->a.canon_taps; cv.w = L.canon;
        cv.row_slot = s->row_slot; cv.row_pos = s->row_pos; cv.row_k = s->row_k;
        cv.state = s->state; cv.slot_stride = s->slot_state; cv.state_off = s->canon_off[r];
        cv.residual = 1; cv.silu = 0;
        cv.out = s->y; cv.ld_out = W; cv.out_bf = s->y_bf;
        cv.entries = s->d_ent; cv.n_entries = s->n_ent;
        QIE_TRY(lay::causal_conv_advance(cv, T, st));
    }
    switch (L.d.mixer) {
        case QIE_MIXER_MINGRU: QIE_TRY(enq_mingru_mixer(b, r, T)); break;
        case QIE_MIXER_LATENT_ATTENTION: QIE_TRY(enq_latent_mixer(b, r, T)); break;
        case QIE_MIXER_CHANNEL_DELTA: QIE_TRY(enq_delta_mixer(b, r, T)); break;
        default: QIE_TRY(enq_gqa_mixer(b, r, T)); break;
    }
    const bool has_ff = L.d.ff_kind != QIE_FF_NONE;
    const bool last = r + 1 == (int)m->runs.size();
    // several rows: the kept stream of a run is the rows' sum, an extra output of the run's last kernel
    const bool fuse_next = !last && (n > 0 || !s->keep_on);
    const LayerDev* N = last ? nullptr : &m->L[m->runs[r + 1].layer];
    const float* next_w = fuse_next ? N->n1 : nullptr;
    const float* next_in = fuse_next ? N->hc_in[0] : nullptr;
    float* sum = n > 0 ? (s->keep_on && s->keep ? s->keep + (int64_t)r * plane : last ? s->x : nullptr) : nullptr;
    if (has_ff) {
        QIE_TRY(step(s->mix, 0, L.hc_in[1], L.n2, false, nullptr));
        QIE_TRY(enq_ff(b, m->runs[r].layer, T));
        QIE_TRY(step(s->ffo, 1, next_in, next_w, true, sum));
    } else {
        QIE_TRY(step(s->mix, 0, next_in, next_w, true, sum));
    }
    *next_ready = fuse_next;
    if (n > 0) {
        if (last && sum != s->x) QIE_HIP(hipMemcpyAsync(s->x, sum, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    } else if (s->keep_on && s->keep) {
        QIE_HIP(hipMemcpyAsync(s->keep + (int64_t)r * plane, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    }
    return 0;
}

// Sandwich blocks: the stream x lives in plane 1 of the stack, the embedding rows stay in plane
// 0.  h_ready: the run's normed input is already in s->y (the previous run's last kernel made
// it).  The last kernel of the run also makes the next run's input unless the streams are kept.
static int enq_run_sandwich(qie_batch* b, int r, int T, bool h_ready, bool* next_ready) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[m->runs[r].layer];
    LayeredBatch* s = b->lb;
    const int W = m->a.width;
    hipStream_t st = e->stream;
    const int64_t plane = s->cap * W;
    float* x0 = s->stack;
    float* x = s->stack + plane;
    const float eps = m->a.norm_eps;
    if (!h_ready) QIE_TRY(lay::add_norm(x, x, nullptr, nullptr, m->runs[r].add_embed ? x0 : nullptr, L.n1, s->y, s->y_bf, T, W, eps, st));
    QIE_REQUIRE(L.d.mixer != QIE_MIXER_LATENT_ATTENTION, "sandwich blocks: latent attention is not wired to them");
    QIE_TRY(enq_gqa_mixer(b, r, T));
    const bool has_ff = L.d.ff_kind != QIE_FF_NONE;
    const bool last = r + 1 == (int)m->runs.size();
    const bool fuse_next = !last && !s->keep_on;
    const LayerDev* N = last ? nullptr : &m->L[m->runs[r + 1].layer];
    const float* nx_add = fuse_next && m->runs[r + 1].add_embed ? x0 : nullptr;
    if (has_ff) {
        QIE_TRY(lay::add_norm(x, x, s->mix, L.n1b, nullptr, L.n2, s->y, s->y_bf, T, W, eps, st));
        QIE_TRY(enq_ff(b, m->runs[r].layer, T));
        QIE_TRY(lay::add_norm(x, x, s->ffo, L.n2b, nx_add, fuse_next ? N->n1 : nullptr, s->y, s->y_bf, T, W, eps, st));
    } else {
        QIE_TRY(lay::add_norm(x, x, s->mix, L.n1b, nx_add, fuse_next ? N->n1 : nullptr, s->y, s->y_bf, T, W, eps, st));
    }
    *next_ready = fuse_next;
    if (s->keep_on && s->keep)
        QIE_HIP(hipMemcpyAsync(s->keep + (int64_t)r * plane, x, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    return 0;
}

static int enq_layer(qie_batch* b, int i, const float* xin, const uint16_t* xin_bf, int T, const float** xout,
                     const uint16_t** xout_bf) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    const LayerDev& L = m->L[i];
    LayeredBatch* s = b->lb;
    const int W = m->a.width;
    hipStream_t st = e->stream;
    const int64_t plane = s->cap * W;
    float* result = s->stack + (int64_t)(i + 1) * plane;
    QIE_TRY(enq_input_proj(b, i, xin, T, xin_bf));
    QIE_TRY(enq_latent_post(b, i, T));
    QIE_TRY(enq_absorb(b, i, T));
    QIE_TRY(enq_attention(b, i, T));
    QIE_TRY(enq_mixer_out(b, i, T));
    const bool has_ff = L.d.ff_kind != QIE_FF_NONE;
    QIE_TRY(lay::postnorm_add(xin, s->mix, has_ff ? s->y : result, has_ff ? s->y_bf : nullptr, T, W, L.g1, m->a.norm_eps, st));
    if (has_ff) {
        QIE_TRY(enq_ff(b, i, T));
        QIE_TRY(lay::postnorm_add(s->y, s->ffo, result, nullptr, T, W, L.g2, m->a.norm_eps, st));
    }
    if (m->a.depth_mix) {
        QIE_TRY(lay::depth_mix(s->stack, plane, L.dwa, i + 2, s->x, s->x_bf, (int64_t)T * W, st));
        *xout = s->x;
        *xout_bf = s->x_bf;
    } else {
        *xout = result;
        *xout_bf = nullptr;
    }
    if (s->keep_on && s->keep)
        QIE_HIP(hipMemcpyAsync(s->keep + (int64_t)i * plane, *xout, (size_t)T * W * 4, hipMemcpyDeviceToDevice, st));
    return 0;
}

static int enq_forward(qie_batch* b, int T, int n_want) {
    const qie_engine* e = b->e;
    const LayeredModel* m = e->lm;
    LayeredBatch* s = b->lb;
    const int W = m->a.width;
    const float* x = s->stack;
    const float w_one = m->a.block == QIE_BLOCK_PRENORM ? m->a.norm_offset : 1.f;
    if (m->a.block == QIE_BLOCK_PRENORM) {
        // one residual row: plane 1; several: planes 0 .. streams - 1, all equal to the embedding output
        const int n = m->a.streams;
        const int64_t plane = s->cap * W;
        float* xs = n > 0 ? s->stack : s->stack + plane;
        float* raw = m->a.embed_norm ? s->mix : xs;
        QIE_TRY(lay::embed_rows(m->embed, m->f32, s->tok, raw, nullptr, T, W, m->a.vocab, e->stream, m->a.embed_scale,
                                m->a.pos_embed == QIE_POS_SINUSOID ? s->row_pos : nullptr, m->pos_freq));
        if (m->a.embed_norm)   // the normed rows go to every stream's plane
            QIE_TRY(lay::add_norm(raw, raw, nullptr, nullptr, nullptr, m->w_embed, xs, nullptr, T, W, m->a.norm_eps, e->stream,
                                  m->a.norm_offset, std::max(n, 1), plane));
        else
            for (int k = 1; k < n; k++)
                QIE_HIP(hipMemcpyAsync(xs + k * plane, xs, (size_t)T * W * 4, hipMemcpyDeviceToDevice, e->stream));
        bool ready = false;
        for (int r = 0; r < (int)m->runs.size(); r++) QIE_TRY(enq_run_prenorm(b, r, T, ready, &ready));
        x = n > 0 ? s->x : xs;
    } else if (m->a.block == QIE_BLOCK_SANDWICH) {
        // the embedding rows stay in plane 0 only when a repeated group adds them again
        float* xs = s->stack + s->cap * W;
        QIE_TRY(lay::embed_rows(m->embed, m->f32, s->tok, m->loops ? s->stack : xs, nullptr, T, W, m->a.vocab, e->stream));
        const LayerDev& L0 = m->L[m->runs[0].layer];
        QIE_TRY(lay::add_norm(xs, m->loops ? s->stack : xs, nullptr, nullptr, nullptr, L0.n1, s->y, s->y_bf, T, W, m->a.norm_eps,
                              e->stream));
        bool ready = true;
        for (int r = 0; r < (int)m->runs.size(); r++) QIE_TRY(enq_run_sandwich(b, r, T, ready, &ready));
        x = xs;
    } else {
        QIE_TRY(lay::embed_rows(m->embed, m->f32, s->tok, s->stack, s->x_bf, T, W, m->a.vocab, e->stream));
        const uint16_t* x_bf = s->x_bf;
        for (int i = 0; i < m->a.n_layers; i++) QIE_TRY(enq_layer(b, i, x, x_bf, T, &x, &x_bf));
    }
    if (n_want > 0) {
        QIE_TRY(lay::final_rows(x, s->want, s->xn, s->xn_bf, n_want, W, m->g_final, m->w_final, m->a.norm_eps, e->stream, w_one));
        QIE_TRY(dense(b, s->xn, W, m->head, s->logits, m->a.vocab, n_want, m->a.vocab, W, s->xn_bf));
    }
    return 0;
}

static void drop_graphs(LayeredBatch* s) {
    for (auto& g : s->graphs)
        if (g.second.second) hipGraphExecDestroy(g.second.second);
    s->graphs.clear();
}

static void lb_free(LayeredBatch* s) {
    drop_graphs(s);   // captured launches hold these buffers' addresses
    void* ps[] = {s->stack, s->x, s->proj, s->qabs, s->olat, s->ov, s->mix, s->y, s->gu, s->act, s->ffo, s->xg, s->yd, s->score,
                  s->row_slot, s->row_pos, s->tok, s->sel, s->cnt, s->off, s->slot_of, s->keep, s->abf,
                  s->x_bf, s->y_bf, s->ov_bf, s->act_bf, s->xg_bf, s->pre, s->aux, s->row_k, s->dw};
    for (void* p : ps)
        if (p) hipFree(p);
    s->stack = s->x = s->proj = s->qabs = s->olat = s->ov = s->mix = s->y = s->gu = s->act = s->ffo = s->xg = s->yd = s->score =
        s->keep = nullptr;
    s->abf = s->x_bf = s->y_bf = s->ov_bf = s->act_bf = s->xg_bf = nullptr;
    s->row_slot = s->row_pos = s->tok = s->sel = s->cnt = s->off = s->slot_of = s->row_k = nullptr;
    s->pre = s->aux = s->dw = nullptr;
    s->cap = 0;
}


// Small steps replay a captured graph of their shape; other steps, and the first run of a shape,
// enqueue eagerly.
static int run_forward(qie_batch* b, int T, int n_want) {
    qie_engine* e = b->e;
    LayeredBatch* s = b->lb;
    const LayeredModel* m = e->lm;
    bool can = e->opts.use_graph && T <= 16 && !s->keep_on;
    for (const LayerDev& L : m->L)
        if (L.d.ff_kind == QIE_FF_MOE && (int64_t)T * L.d.top >= kMoeSyncRows) can = false;   // host round trip inside
    if (!can) return enq_forward(b, T, n_want);
    std::vector<int> key{T, n_want, s->n_ent, s->n_qgroups};
    for (const auto& g : s->groups) {
        key.push_back(g.first);
        key.push_back(g.second.first);
        key.push_back((int)g.second.second);
    }
    auto& slot = s->graphs[key];
    slot.first++;
    if (slot.first == 1) return enq_forward(b, T, n_want);   // allocations and lazy attributes happen here
    if (!slot.second && slot.first == 2) {
        hipGraph_t graph = nullptr;
        QIE_HIP(hipStreamBeginCapture(e->stream, hipStreamCaptureModeThreadLocal));
        const int rc = enq_forward(b, T, n_want);
        const hipError_t he = hipStreamEndCapture(e->stream, &graph);
        if (rc || he != hipSuccess || !graph) {
            if (graph) hipGraphDestroy(graph);
            (void)hipGetLastError();
            if (rc) return rc;
            return enq_forward(b, T, n_want);   // this shape stays eager
        }
        hipGraphExec_t ex = nullptr;
        const hipError_t hi = hipGraphInstantiate(&ex, graph, nullptr, nullptr, 0);
        hipGraphDestroy(graph);
        if (hi != hipSuccess || !ex) {
            (void)hipGetLastError();
            return enq_forward(b, T, n_want);
        }
        slot.second = ex;
    }
    if (slot.second) {
        QIE_HIP(hipGraphLaunch(slot.second, e->stream));
        s->graph_replays++;
        return 0;
    }
    return enq_forward(b, T, n_want);
}

static int ensure_rows(qie_batch* b, int64_t T) {
    LayeredBatch* s = b->lb;
    const LayeredModel* m = b->e->lm;
    if (T > s->cap) {
        QIE_HIP(hipStreamSynchronize(b->e->stream));
        lb_free(s);
        const int64_t cap = (T + 63) / 64 * 64, W = m->a.width, L = m->a.n_layers;
        int rc = 0;
        auto A = [&](void** p, int64_t elems, size_t sz = 4) {
            if (!rc) rc = dmalloc(p, (size_t)elems * sz);
        };
        A((void**)&s->stack, (m->a.depth_mix ? L + 1 : std::max<int64_t>(2, m->a.streams)) * cap * W);
        A((void**)&s->pre, cap * std::max<int64_t>(s->m_pre, 1));
        A((void**)&s->aux, cap * std::max<int64_t>(s->m_aux, 1));
        if (s->m_dw > 0) A((void**)&s->dw, cap * s->m_dw);
        A((void**)&s->row_k, cap);
        A((void**)&s->x, cap * W);
        A((void**)&s->proj, cap * s->m_in);
        A((void**)&s->qabs, cap * std::max<int64_t>(s->m_hr, 1));
        A((void**)&s->olat, cap * std::max<int64_t>(s->m_hr, 1));
        A((void**)&s->ov, cap * s->m_hv);
        A((void**)&s->mix, cap * W);
        A((void**)&s->y, cap * W);
        A((void**)&s->gu, cap * std::max<int64_t>(s->m_gu, 1));
        A((void**)&s->act, cap * std::max<int64_t>(s->m_act, 1));
        A((void**)&s->ffo, cap * W);
        A((void**)&s->xg, cap * std::max<int64_t>(s->m_top, 1) * W);
        A((void**)&s->yd, cap * std::max<int64_t>(s->m_top, 1) * W);
        A((void**)&s->score, cap * std::max<int64_t>(s->m_top, 1));
        A((void**)&s->sel, cap * std::max<int64_t>(s->m_top, 1));
        A((void**)&s->slot_of, cap * std::max<int64_t>(s->m_top, 1));
        A((void**)&s->cnt, s->m_e + 1);
        A((void**)&s->off, s->m_e + 2);
        A((void**)&s->row_slot, cap);
        A((void**)&s->row_pos, cap);
        A((void**)&s->tok, cap);
        if (!m->f32) {
            A((void**)&s->abf, cap * s->m_abf + 64, 2);
            A((void**)&s->x_bf, cap * W, 2);
            A((void**)&s->y_bf, cap * W, 2);
            A((void**)&s->ov_bf, cap * s->m_hv, 2);
            A((void**)&s->act_bf, cap * std::max<int64_t>(s->m_act, 1), 2);
            A((void**)&s->xg_bf, cap * std::max<int64_t>(s->m_top, 1) * W, 2);
        }
        if (s->keep_on) A((void**)&s->keep, (int64_t)m->runs.size() * cap * W);
        if (rc) return rc;
        s->cap = cap;
    }
    if (s->keep_on && !s->keep) drop_graphs(s);
    if (s->keep_on && !s->keep) QIE_TRY(dmalloc((void**)&s->keep, m->runs.size() * s->cap * m->a.width * 4));
    if (T > s->h_stage_rows) {
        if (s->h_stage) hipHostFree(s->h_stage);
        s->h_stage = nullptr;
        const int64_t rows = (T + 255) / 256 * 256;
        QIE_HIP(hipHostMalloc((void**)&s->h_stage, (size_t)rows * 4 * 4, hipHostMallocDefault));
        s->h_stage_rows = rows;
    }
    return 0;
}

static int ensure_want(qie_batch* b, int64_t n) {
    LayeredBatch* s = b->lb;
    const LayeredModel* m = b->e->lm;
    if (n <= s->want_cap) return 0;
    QIE_HIP(hipStreamSynchronize(b->e->stream));
    drop_graphs(s);
    void* ps[] = {s->want, s->xn, s->logits, s->logits_bf, s->d_ids, s->d_step, s->xn_bf};
    for (void* p : ps)
        if (p) hipFree(p);
    s->xn_bf = nullptr;
    s->want = nullptr; s->xn = nullptr; s->logits = nullptr; s->logits_bf = nullptr; s->d_ids = nullptr; s->d_step = nullptr;
    s->want_cap = 0;
    const int64_t cap = (n + 15) / 16 * 16, V = m->a.vocab;
    QIE_TRY(dmalloc((void**)&s->want, cap * 4));
    QIE_TRY(dmalloc((void**)&s->xn, cap * m->a.width * 4));
    if (!m->f32) QIE_TRY(dmalloc((void**)&s->xn_bf, cap * m->a.width * 2));
    QIE_TRY(dmalloc((void**)&s->logits, cap * V * 4));
    QIE_TRY(dmalloc((void**)&s->logits_bf, cap * V * 2));
    QIE_TRY(dmalloc((void**)&s->d_ids, cap * 4));
    QIE_TRY(dmalloc((void**)&s->d_step, cap * 4));
    if (b->samp_ws) hipFree(b->samp_ws);
    b->samp_ws = nullptr;
    QIE_TRY(dmalloc(&b->samp_ws, (size_t)qie_sample_workspace_bytes(cap, V)));
    s->want_cap = cap;
    return 0;
}

int layered_batch_create(qie_engine* e, int32_t batch, int32_t max_ctx, int32_t page_tokens, int32_t n_pages, qie_batch** out) {
    LayeredModel* m = e->lm;
    QIE_REQUIRE(m->final, "qie_batch_create_paged: the layered engine's weights are not finalized");
    QIE_REQUIRE(out && batch > 0 && batch <= 4096 && max_ctx > 1, "qie_batch_create_paged: bad arguments");
    QIE_REQUIRE(max_ctx <= e->opts.max_ctx, "qie_batch_create_paged: max_ctx %d > engine max_ctx %d", max_ctx, e->opts.max_ctx);
    if (page_tokens == 0) page_tokens = 64;
    QIE_REQUIRE(page_tokens >= 16 && (page_tokens & (page_tokens - 1)) == 0,
                "qie_batch_create_paged: page_tokens %d must be a power of two >= 16 (layered engines)", page_tokens);
    QIE_REQUIRE(n_pages == 0 || n_pages >= 2, "qie_batch_create_paged: need the scratch page and one more");
    qie_batch* b = new qie_batch();
    LayeredBatch* s = new LayeredBatch();
    b->e = e;
    b->lb = s;
    b->B = batch;
    b->max_ctx = max_ctx;
    b->page_tokens = page_tokens;
    b->max_pages = (max_ctx + page_tokens - 1) / page_tokens;
    b->n_pages = n_pages > 0 ? n_pages : batch * b->max_pages + 1;
    const int n_runs = (int)m->runs.size();
    s->layer_off.assign(n_runs, 0);
    s->v_off.assign(n_runs, 0);
    s->state_off.assign(n_runs, 0);
    s->conv_off.assign(n_runs, 0);
    s->canon_off.assign(n_runs, 0);
    // bf16 caches whose every layer fits the matrix-core attention carry, after the rows of a
    // caching layer, the key-interleaved copy of c (R more elements per token)
    s->il_of.assign(m->a.n_layers, 0);
    for (int i = 0; i < m->a.n_layers; i++) {
        const qie_layer_desc& d = m->L[i].d;
        if (!m->f32 && d.mixer == QIE_MIXER_LATENT_ATTENTION && page_tokens % 16 == 0 &&
            lay::latent_attention_mfma_fits(d.kv_rank, d.rot_dim))
            s->il_of[i] = 1;
    }
    for (int i = 0; i < m->a.n_layers; i++) {
        if (m->L[i].d.mixer == QIE_MIXER_LATENT_ATTENTION) s->il_of[i] = s->il_of[m->L[i].cache_layer];
        if (s->il_of[i]) s->interleaved = true;
    }
    // bf16 grouped-query caches whose every layer fits the matrix-core attention store V transposed
    s->vt_of.assign(n_runs, 0);
    for (int r = 0; r < n_runs; r++) {
        const qie_layer_desc& d = m->L[m->runs[r].layer].d;
        if (d.mixer != QIE_MIXER_GQA && d.mixer != QIE_MIXER_GQA_RECURRENT) continue;
        if (!m->f32 && lay::gqa_attention_mfma_fits(d.gqa.dim, d.gqa.vdim, page_tokens)) s->vt_of[r] = 1, s->v_transposed = true;
        s->m_vd = std::max<int64_t>(s->m_vd, d.gqa.vdim);
    }
    int64_t off = 0;
    for (int r = 0; r < n_runs; r++) {
        const int i = m->runs[r].layer;
        const qie_layer_desc& d = m->L[i].d;
        if (m->a.canon_taps > 1) {   // the last taps - 1 normed mixer inputs of every run
            s->canon_off[r] = s->slot_state;
            s->slot_state += (int64_t)(m->a.canon_taps - 1) * m->a.width;
        }
        if (d.mixer == QIE_MIXER_CHANNEL_DELTA) {
            // no cache rows; per slot the heads' states and the short convolutions' last inputs
            const qie_delta_desc& c = d.delta;
            const int64_t C = 2 * (int64_t)c.kv_heads * c.dim + (int64_t)c.heads * c.vdim;
            s->state_off[r] = s->slot_state;
            s->slot_state += (int64_t)c.heads * c.dim * c.vdim;
            s->conv_off[r] = s->slot_state;
            s->slot_state += (int64_t)(c.conv - 1) * C;
            s->m_in = std::max<int64_t>(s->m_in, m->L[i].n_in);
            s->m_pre = std::max<int64_t>(s->m_pre, C);
            s->m_hr = std::max<int64_t>({s->m_hr, (int64_t)c.heads * c.dim, (int64_t)c.heads * c.vdim});
            s->m_aux = std::max<int64_t>(s->m_aux, (int64_t)c.heads * c.vdim);
            s->m_dw = std::max<int64_t>(s->m_dw, (int64_t)c.heads * c.dim);
            s->m_state = std::max<int64_t>(s->m_state, (int64_t)c.heads * c.dim * c.vdim);
            s->m_hd = std::max<int64_t>(s->m_hd, (int64_t)c.heads * c.dim * c.dim);
            s->m_hv = std::max<int64_t>(s->m_hv, (int64_t)c.heads * c.vdim);
            s->m_abf = std::max<int64_t>({s->m_abf, (int64_t)m->a.width, (int64_t)c.heads * c.vdim});
        } else if (d.mixer == QIE_MIXER_MINGRU) {
            // no cache rows; `width` state elements per slot
            const int64_t n = d.mingru.width;
            s->state_off[r] = s->slot_state;
            s->slot_state += n;
            s->m_state = std::max<int64_t>(s->m_state, n);
            s->m_hd = std::max<int64_t>(s->m_hd, n);
            s->m_in = std::max<int64_t>(s->m_in, m->L[i].n_in);
            s->m_hv = std::max<int64_t>(s->m_hv, n);
            s->m_abf = std::max<int64_t>({s->m_abf, (int64_t)m->a.width, n});
        } else if (d.mixer != QIE_MIXER_LATENT_ATTENTION) {
            // K rows, then V rows of this run; one state per slot for the recurrence
            const qie_gqa_desc& a = d.gqa;
            s->layer_off[r] = off;
            off += (int64_t)page_tokens * a.kv_heads * a.dim;
            s->v_off[r] = off;
            off += (int64_t)page_tokens * a.kv_heads * a.vdim;
            const int64_t rv = d.mixer == QIE_MIXER_GQA_RECURRENT ? (int64_t)d.rec.heads * d.rec.vdim : 0;
            if (rv) {
                s->state_off[r] = s->slot_state;
                s->slot_state += (int64_t)d.rec.heads * d.rec.dim * d.rec.vdim;
                s->m_state = std::max<int64_t>(s->m_state, (int64_t)d.rec.heads * d.rec.dim * d.rec.vdim);
                s->m_hd = std::max<int64_t>(s->m_hd, (int64_t)d.rec.heads * d.rec.dim);
            }
            s->m_in = std::max<int64_t>(s->m_in, m->L[i].n_in);
            s->m_hr = std::max<int64_t>(s->m_hr, rv);
            s->m_hv = std::max<int64_t>(s->m_hv, m->L[i].n_cat);
            s->m_abf = std::max<int64_t>({s->m_abf, (int64_t)m->a.width, (int64_t)m->L[i].n_cat});
        }
    }
    for (int i = 0; i < m->a.n_layers; i++) {
        const qie_layer_desc& d = m->L[i].d;
        const int64_t k = d.ff_kind == QIE_FF_MOE ? d.top : 1;
        if (d.mixer != QIE_MIXER_LATENT_ATTENTION) {
            if (d.ff_kind != QIE_FF_NONE) {
                s->m_gu = std::max<int64_t>(s->m_gu, k * 2 * d.ff);
                s->m_act = std::max<int64_t>(s->m_act, k * d.ff);
                s->m_abf = std::max<int64_t>(s->m_abf, k * std::max<int64_t>(d.ff, m->a.width));
            }
            if (d.ff_kind == QIE_FF_MOE) {
                s->m_top = std::max<int64_t>(s->m_top, d.top);
                s->m_e = std::max<int64_t>(s->m_e, d.experts + (d.router == QIE_ROUTER_SOFTMAX_ALL ? d.identity : 0));
            }
            continue;
        }
        if (d.kv_from < 0) {
            s->layer_off[i] = off;
            off += (int64_t)page_tokens * (d.kv_rank + d.rot_dim + (s->il_of[i] ? d.kv_rank : 0));
        }
        const int64_t H = d.heads;
        s->m_in = std::max<int64_t>(s->m_in, m->L[i].n_in);
        s->m_pre = std::max<int64_t>(s->m_pre, m->L[i].n_pre);
        s->m_abf = std::max<int64_t>(s->m_abf, d.q_rank);
        s->m_hr = std::max<int64_t>(s->m_hr, H * d.kv_rank);
        s->m_r = std::max<int64_t>(s->m_r, d.kv_rank);
        s->m_hv = std::max<int64_t>(s->m_hv, H * d.vdim);
        if (d.ff_kind != QIE_FF_NONE) {
            s->m_gu = std::max<int64_t>(s->m_gu, k * 2 * d.ff);
            s->m_act = std::max<int64_t>(s->m_act, k * d.ff);
        }
        s->m_abf = std::max<int64_t>({s->m_abf, (int64_t)m->a.width, H * (d.dim + d.rot_dim), H * d.kv_rank, H * d.vdim,
                                      d.ff_kind == QIE_FF_NONE ? 0 : k * std::max<int64_t>(d.ff, m->a.width)});
        if (d.ff_kind == QIE_FF_MOE) {
            s->m_top = std::max<int64_t>(s->m_top, d.top);
            s->m_e = std::max<int64_t>(s->m_e, d.experts);
        }
    }
    b->seq_stride = off;   // elements per page
    b->h_table.assign((size_t)batch * b->max_pages, 0);
    for (int p = b->n_pages - 1; p >= 1; p--) b->free_pages.push_back(p);
    b->held.assign(batch, 0);
    b->idle.assign(batch, 1);
    b->h_pos.assign(batch, 0);
    b->table_dirty = true;
    const size_t pool = (size_t)b->n_pages * off * m->esz();
    int rc = dmalloc((void**)&b->kc, pool);
    if (!rc) rc = dmalloc((void**)&b->d_table, b->h_table.size() * 4);
    if (!rc && s->slot_state > 0) rc = dmalloc((void**)&s->state, (size_t)batch * s->slot_state * 4);
    if (!rc) {
        hipError_t he = hipMemsetAsync(b->kc, 0, pool, e->stream);
        if (he == hipSuccess && s->state) he = hipMemsetAsync(s->state, 0, (size_t)batch * s->slot_state * 4, e->stream);
        if (he == hipSuccess) he = hipStreamSynchronize(e->stream);
        if (he != hipSuccess) rc = fail((int)he, "batch init: %s", hipGetErrorString(he));
    }
    if (!rc) rc = flush_table(b);
    if (!rc) {
        hipError_t he = hipEventCreateWithFlags(&s->ev_fork, hipEventDisableTiming);
        for (int i = 0; i < LayeredBatch::kSide && he == hipSuccess; i++) {
            he = hipStreamCreateWithFlags(&s->side[i], hipStreamNonBlocking);
            if (he == hipSuccess) he = hipEventCreateWithFlags(&s->ev_join[i], hipEventDisableTiming);
        }
        if (he != hipSuccess) rc = fail((int)he, "batch init (side streams): %s", hipGetErrorString(he));
    }
    if (rc) {
        qie_batch_destroy(b);
        return rc;
    }
    *out = b;
    return 0;
}

void layered_batch_destroy(qie_batch* b) {
    LayeredBatch* s = b->lb;
    if (!s) return;
    lb_free(s);
    void* ps[] = {s->want, s->xn, s->logits, s->logits_bf, s->d_ids, s->d_step, s->d_groups, s->part_o, s->part_ml, s->xn_bf,
                  s->state, s->d_ent, s->d_qgroups, s->gpart_o, s->gpart_ml, s->d_chunks, s->d_spans, s->s_loc, s->s_in, s->s_decay};
    for (void* p : ps)
        if (p) hipFree(p);
    if (s->h_stage) hipHostFree(s->h_stage);
    for (int i = 0; i < LayeredBatch::kSide; i++) {
        if (s->side[i]) hipStreamSynchronize(s->side[i]);
        if (s->ev_join[i]) hipEventDestroy(s->ev_join[i]);
        if (s->side[i]) hipStreamDestroy(s->side[i]);
    }
    if (s->ev_fork) hipEventDestroy(s->ev_fork);
    delete s;
    b->lb = nullptr;
}

}  // namespace qie

using namespace qie;

extern "C" {

int qie_engine_create_layered(const qie_arch_desc* arch, const qie_engine_opts* opts, qie_engine** out) {
    QIE_REQUIRE(arch && out && arch->layers, "qie_engine_create_layered: bad arguments");
    QIE_REQUIRE(arch->n_layers > 0 && arch->width > 0 && arch->vocab > 0 && arch->norm_eps >= 0.f,
                "qie_engine_create_layered: invalid sizes");
    QIE_REQUIRE(!opts || !opts->tp_comm, "qie_engine_create_layered: layered engines run on one device");
    QIE_REQUIRE(!opts || (!opts->weight_fp8 && !opts->prefill_fp8), "qie_engine_create_layered: fp8 weights are not covered");
    QIE_REQUIRE(arch->block >= QIE_BLOCK_POSTNORM_GAIN && arch->block <= QIE_BLOCK_PRENORM, "qie_engine_create_layered: block %d",
                arch->block);
    QIE_REQUIRE(arch->pos_embed == QIE_POS_NONE || arch->pos_embed == QIE_POS_SINUSOID, "qie_engine_create_layered: positions %d",
                arch->pos_embed);
    QIE_REQUIRE((arch->pos_embed == QIE_POS_NONE && (arch->embed_scale == 0.f || arch->embed_scale == 1.f)) ||
                    arch->block == QIE_BLOCK_PRENORM,
                "qie_engine_create_layered: scaled embeddings and position vectors go with the pre-norm block");
    QIE_REQUIRE(arch->block == QIE_BLOCK_POSTNORM_GAIN || !arch->depth_mix,
                "qie_engine_create_layered: depth-weighted residuals go with the post-norm block");
    const bool loops = arch->loop_times > 1 && arch->loop_stop > arch->loop_start;
    QIE_REQUIRE(!loops || (arch->loop_start >= 0 && arch->loop_stop <= arch->n_layers && arch->loop_times <= 64),
                "qie_engine_create_layered: repeated group [%d, %d) x %d of %d layers", arch->loop_start, arch->loop_stop,
                arch->loop_times, arch->n_layers);
    QIE_REQUIRE(!loops || arch->block == QIE_BLOCK_SANDWICH, "qie_engine_create_layered: repeated groups go with the sandwich block");
    QIE_REQUIRE(arch->streams >= 0 && arch->streams <= 32 && arch->canon_taps >= 0 && arch->canon_taps <= 64,
                "qie_engine_create_layered: %d residual streams (at most 32), %d input taps (at most 64)", arch->streams, arch->canon_taps);
    QIE_REQUIRE(arch->block == QIE_BLOCK_PRENORM || (arch->streams == 0 && arch->canon_taps == 0 && !arch->embed_norm &&
                                                     arch->norm_offset == 0.f),
                "qie_engine_create_layered: residual streams, the input convolution, the embedding norm and the norm offset "
                "go with the pre-norm block");
    for (int i = 0; i < arch->n_layers; i++) {
        const qie_layer_desc& d = arch->layers[i];
        QIE_REQUIRE(d.ff_kind >= QIE_FF_NONE && d.ff_kind <= QIE_FF_MOE, "layer %d: unknown feed-forward %d", i, d.ff_kind);
        QIE_REQUIRE(d.ff_kind == QIE_FF_NONE || d.ff > 0, "layer %d: feed-forward size", i);
        QIE_REQUIRE(d.ff_kind != QIE_FF_MOE || (d.experts > 0 && d.top > 0 && d.top <= d.experts + std::max(d.identity, 0)),
                    "layer %d: %d of %d experts", i, d.top, d.experts + std::max(d.identity, 0));
        QIE_REQUIRE(d.router >= QIE_ROUTER_SIGMOID_IN && d.router <= QIE_ROUTER_SOFTMAX_ALL, "layer %d: router %d", i, d.router);
        QIE_REQUIRE(d.ff_act >= QIE_ACT_SILU_GATED && d.ff_act <= QIE_ACT_GELU_TANH_GATED, "layer %d: activation %d", i, d.ff_act);
        if (d.ff_kind == QIE_FF_MOE && d.router == QIE_ROUTER_SOFTMAX_ALL) {
            const int n = d.experts + d.identity;
            QIE_REQUIRE(d.identity >= 0 && d.groups >= 1 && n % d.groups == 0 && d.groups_keep >= 1 && d.groups_keep <= d.groups &&
                            d.top <= d.groups_keep * (n / d.groups),
                        "layer %d: %d + %d router outputs in %d groups, %d kept, top %d", i, d.experts, d.identity, d.groups,
                        d.groups_keep, d.top);
        } else {
            QIE_REQUIRE(d.identity == 0, "layer %d: identity experts go with the grouped softmax router", i);
        }
        if (d.mixer == QIE_MIXER_MINGRU) {
            QIE_REQUIRE(arch->block == QIE_BLOCK_PRENORM, "layer %d: this mixer is wired to the pre-norm block", i);
            QIE_REQUIRE(d.mingru.width > 0, "layer %d: minGRU width", i);
            continue;
        }
        if (d.mixer == QIE_MIXER_CHANNEL_DELTA) {
            const qie_delta_desc& c = d.delta;
            QIE_REQUIRE(arch->block == QIE_BLOCK_PRENORM, "layer %d: this mixer is wired to the pre-norm block", i);
            QIE_REQUIRE(c.heads > 0 && c.kv_heads > 0 && c.heads % c.kv_heads == 0 && c.dim > 0 && c.dim <= 512 && c.vdim > 0 &&
                            c.conv >= 1 && c.conv <= 64 && c.rank_a >= 0 && c.rank_g >= 0,
                        "layer %d: delta rule with %d heads over %d key heads of %d (at most 512) / %d, %d taps", i, c.heads, c.kv_heads,
                        c.dim, c.vdim, c.conv);
            continue;
        }
        if (d.mixer == QIE_MIXER_GQA || d.mixer == QIE_MIXER_GQA_RECURRENT) {
            const qie_gqa_desc& a = d.gqa;
            QIE_REQUIRE(arch->block == QIE_BLOCK_SANDWICH || (arch->block == QIE_BLOCK_PRENORM && d.mixer == QIE_MIXER_GQA),
                        "layer %d: this mixer is wired to the sandwich block (alone: also the pre-norm block)", i);
            QIE_REQUIRE(a.weights == QIE_WEIGHTS_SOFTMAX || a.weights == QIE_WEIGHTS_SIGMOID, "layer %d: attention weights %d", i,
                        a.weights);
            QIE_REQUIRE(a.q_temp_every >= 0, "layer %d: query temperature every %d", i, a.q_temp_every);
            QIE_REQUIRE(a.heads > 0 && a.kv_heads > 0 && a.heads % a.kv_heads == 0 && a.dim > 0 && a.vdim > 0,
                        "layer %d: %d query heads over %d key heads of %d / %d", i, a.heads, a.kv_heads, a.dim, a.vdim);
            QIE_REQUIRE(a.qk_norm >= QIE_QKNORM_NONE && a.qk_norm <= QIE_QKNORM_PLAIN, "layer %d: q / k norm %d", i, a.qk_norm);
            QIE_REQUIRE(a.rot_dims >= 0 && a.rot_dims % 2 == 0 && a.rot_dims <= a.dim, "layer %d: rotary dims %d of %d", i, a.rot_dims,
                        a.dim);
            QIE_REQUIRE(a.rot_layout == QIE_ROT_HALVES || a.rot_layout == QIE_ROT_INTERLEAVED, "layer %d: rotary layout %d", i,
                        a.rot_layout);
            QIE_REQUIRE((a.rot_dims == 0 && !a.rot_values) || a.rot_base > 0.f, "layer %d: rotary base", i);
            QIE_REQUIRE(!a.rot_values || a.vdim % 2 == 0, "layer %d: turned values need an even vdim", i);
            QIE_REQUIRE(a.mask >= QIE_MASK_CAUSAL && a.mask <= QIE_MASK_CHUNK && (a.mask == QIE_MASK_CAUSAL || a.mask_size > 0),
                        "layer %d: mask %d of size %d", i, a.mask, a.mask_size);
            QIE_REQUIRE(!a.values_are_keys || (a.vdim == a.dim && !a.rot_values), "layer %d: keys as values need vdim == dim", i);
            QIE_REQUIRE(!(a.out_gate && a.head_gate), "layer %d: one output gate, per head or per coordinate", i);
            QIE_REQUIRE(!a.sink || a.weights == QIE_WEIGHTS_SOFTMAX, "layer %d: a sink goes with softmax weights", i);
            QIE_REQUIRE(a.rot_scaling.factor == 0.f || (a.rot_scaling.factor > 0.f && a.rot_scaling.high > a.rot_scaling.low &&
                                                        a.rot_scaling.low >= 0.f && a.rot_scaling.original > 0.f),
                        "layer %d: rotary scaling", i);
            if (d.mixer == QIE_MIXER_GQA_RECURRENT)
                QIE_REQUIRE(d.rec.heads > 0 && d.rec.dim > 0 && d.rec.dim <= 512 && d.rec.vdim > 0, "layer %d: recurrence sizes", i);
            continue;
        }
        QIE_REQUIRE(d.mixer == QIE_MIXER_LATENT_ATTENTION, "layer %d: unknown mixer %d", i, d.mixer);
        QIE_REQUIRE(arch->block == QIE_BLOCK_POSTNORM_GAIN || arch->block == QIE_BLOCK_PRENORM,
                    "layer %d: latent attention is wired to the post-norm and pre-norm blocks", i);
        QIE_REQUIRE(d.heads > 0 && d.dim > 0 && d.rot_dim >= 0 && d.vdim > 0 && d.kv_rank > 0 && d.window >= 0 && d.q_rank >= 0,
                    "layer %d: invalid mixer sizes", i);
        QIE_REQUIRE(d.rot_layout == QIE_ROT_HALVES || d.rot_layout == QIE_ROT_INTERLEAVED, "layer %d: rotary layout %d", i, d.rot_layout);
        QIE_REQUIRE(d.q_rank == 0 || !d.head_gate, "layer %d: latent queries and the head gate are not wired together", i);
        QIE_REQUIRE(d.rot_dims >= 0 && d.rot_dims % 2 == 0 && d.rot_dims <= d.rot_dim, "layer %d: rotary dims %d of %d", i,
                    d.rot_dims, d.rot_dim);
        QIE_REQUIRE(d.rot_dims == 0 || d.rot_base > 0.f, "layer %d: rotary base", i);
        if (d.kv_from >= 0) {
            QIE_REQUIRE(d.kv_from < i, "layer %d: kv_from %d must name an earlier layer", i, d.kv_from);
            const qie_layer_desc& o = arch->layers[d.kv_from];
            QIE_REQUIRE(o.mixer == QIE_MIXER_LATENT_ATTENTION && o.kv_from < 0 && o.kv_rank == d.kv_rank && o.rot_dim == d.rot_dim &&
                            o.rot_dims == d.rot_dims && o.rot_base == d.rot_base && o.rot_layout == d.rot_layout &&
                            memcmp(&o.rot_scaling, &d.rot_scaling, sizeof(qie_rot_scaling)) == 0,
                        "layer %d: the layer it reads its cache from (%d) must own one of the same shape and rotation", i,
                        d.kv_from);
        }
    }
    qie_engine* e = new qie_engine();
    if (opts) e->opts = *opts;
    if (e->opts.max_ctx <= 0) e->opts.max_ctx = 4096;
    e->opts.tp_size = 1;
    e->opts.tp_rank = 0;
    e->sh.tp = 1;
    LayeredModel* m = new LayeredModel();
    e->lm = m;
    m->a = *arch;
    m->descs.assign(arch->layers, arch->layers + arch->n_layers);
    m->a.layers = m->descs.data();
    m->f32 = e->opts.compute_f32 != 0;
    m->L.resize(arch->n_layers);
    for (int i = 0; i < arch->n_layers; i++) {
        m->L[i].d = m->descs[i];
        m->L[i].cache_layer = m->descs[i].kv_from >= 0 ? m->descs[i].kv_from : i;
    }
    m->loops = loops;
    for (int i = 0; i < arch->n_layers; i++) {
        if (loops && i == arch->loop_start) {
            for (int t = 0; t < arch->loop_times; t++)
                for (int j = arch->loop_start; j < arch->loop_stop; j++) m->runs.push_back(LayerRun{j, t > 0 && j == arch->loop_start});
            i = arch->loop_stop - 1;
            continue;
        }
        m->runs.push_back(LayerRun{i, false});
    }
    // informational mirror for qie_engine_spec
    e->spec.n_layers = arch->n_layers;
    e->spec.hidden = arch->width;
    e->spec.vocab = arch->vocab;
    e->spec.rms_eps = arch->norm_eps;
    hipError_t he = hipSetDevice(e->opts.device);
    if (he == hipSuccess) he = hipStreamCreateWithFlags(&e->stream, hipStreamNonBlocking);
    if (he != hipSuccess) {
        qie_engine_destroy(e);
        return fail((int)he, "qie_engine_create_layered: %s", hipGetErrorString(he));
    }
    *out = e;
    return 0;
}

int qie_engine_put_tensor(qie_engine* e, const char* name, const void* host, int32_t dtype, int32_t ndim, const int64_t* shape) {
    QIE_REQUIRE(e && e->lm && name && host && dtype >= 0 && dtype <= 2 && ndim >= 0 && ndim <= 4 && (ndim == 0 || shape),
                "qie_engine_put_tensor: bad arguments (layered engines)");
    QIE_REQUIRE(!e->lm->final, "qie_engine_put_tensor: weights are finalized");
    HostTensor t;
    t.dtype = dtype;
    t.shape.assign(shape, shape + ndim);
    const int64_t n = t.numel();
    QIE_REQUIRE(n >= 0, "qie_engine_put_tensor: bad shape");
    t.data.resize((size_t)n * (dtype == 0 ? 2 : 4));
    memcpy(t.data.data(), host, t.data.size());
    e->lm->host[name] = std::move(t);
    return 0;
}

int qie_engine_finalize_weights(qie_engine* e) {
    QIE_REQUIRE(e && e->lm, "qie_engine_finalize_weights: a layered engine");
    LayeredModel* m = e->lm;
    QIE_REQUIRE(!m->final, "qie_engine_finalize_weights: already done");
    QIE_HIP(hipSetDevice(e->opts.device));
    const int64_t W = m->a.width, V = m->a.vocab;
    LM_GET(te, "embed", V, W);
    QIE_TRY(lm_alloc(m, &m->embed, (size_t)V * W * m->esz()));
    QIE_TRY(lm_upload_rows(m, m->embed, 0, W, *te));
    if (m->a.tied_head) {
        m->head = m->embed;
    } else {
        LM_GET(th, "head", V, W);
        QIE_TRY(lm_alloc(m, &m->head, (size_t)V * W * m->esz()));
        QIE_TRY(lm_upload_rows(m, m->head, 0, W, *th));
    }
    if (m->a.embed_scale == 0.f) m->a.embed_scale = 1.f;
    if (m->a.pos_embed == QIE_POS_SINUSOID) {
        std::vector<double> fr((size_t)(W + 1) / 2);
        for (size_t i = 0; i < fr.size(); i++) fr[i] = std::pow(10000.0, -2.0 * (double)i / (double)W);
        QIE_TRY(lm_alloc(m, (void**)&m->pos_freq, fr.size() * 8));
        QIE_HIP(hipMemcpy(m->pos_freq, fr.data(), fr.size() * 8, hipMemcpyHostToDevice));
    }
    if (m->a.embed_norm) QIE_TRY(lm_vector(m, &m->w_embed, "embed.norm", W));
    if (m->a.block == QIE_BLOCK_SANDWICH || m->a.block == QIE_BLOCK_PRENORM) {
        QIE_TRY(lm_vector(m, &m->w_final, "final.norm", W));
    } else {
        LM_GET(tn, "final.norm");
        m->g_final = host_elem(*tn, 0);
    }
    for (int i = 0; i < m->a.n_layers; i++) QIE_TRY(finalize_layer(e, m, i));
    m->host.clear();
    m->final = true;
    e->have_weights = true;
    return 0;
}

int qie_batch_step(qie_batch* b, int32_t n_entries, const int32_t* slots, const int32_t* counts, const int32_t* tokens,
                   int32_t n_want, const int32_t* want_rows, float* host_logits) {
    QIE_REQUIRE(b && b->lb, "qie_batch_step: a batch of a layered engine");
    QIE_REQUIRE(n_entries > 0 && slots && counts && tokens && n_want >= 0 && (n_want == 0 || want_rows),
                "qie_batch_step: bad arguments");
    qie_engine* e = b->e;
    LayeredBatch* s = b->lb;
    QIE_HIP(hipSetDevice(e->opts.device));
    int64_t T = 0, new_pages = 0;
    std::vector<char> seen(b->B, 0);
    for (int i = 0; i < n_entries; i++) {
        const int sl = slots[i];
        QIE_REQUIRE(sl >= 0 && sl < b->B && !seen[sl], "qie_batch_step: entry %d: slot %d out of range or repeated", i, sl);
        seen[sl] = 1;
        QIE_REQUIRE(counts[i] > 0, "qie_batch_step: entry %d: empty", i);
        const int64_t p0 = b->idle[sl] ? 0 : b->h_pos[sl], p1 = p0 + counts[i];
        QIE_REQUIRE(p1 <= b->max_ctx, "qie_batch_step: slot %d would hold %lld tokens, max_ctx %d", sl, (long long)p1, b->max_ctx);
        const int64_t held = b->idle[sl] ? 0 : b->held[sl];
        new_pages += std::max<int64_t>(0, (p1 + b->page_tokens - 1) / b->page_tokens - held);
        T += counts[i];
    }
    QIE_REQUIRE(new_pages <= (int64_t)b->free_pages.size(), "qie_batch_step: the step needs %lld more pages, %zu free",
                (long long)new_pages, b->free_pages.size());
    for (int i = 0; i < n_want; i++)
        QIE_REQUIRE(want_rows[i] >= 0 && want_rows[i] < T, "qie_batch_step: wanted row %d outside the step's %lld rows",
                    want_rows[i], (long long)T);
    QIE_TRY(ensure_rows(b, T));
    QIE_TRY(ensure_want(b, std::max(n_want, 1)));
    int32_t* hs = s->h_stage;
    const int64_t R = s->h_stage_rows;
    int64_t r = 0;
    for (int i = 0; i < n_entries; i++) {
        const int sl = slots[i];
        if (b->idle[sl]) {
            b->idle[sl] = 0;
            b->h_pos[sl] = 0;
        }
        QIE_TRY(ensure_pages(b, sl, (int64_t)b->h_pos[sl] + counts[i]));
        for (int k = 0; k < counts[i]; k++, r++) {
            hs[r] = sl;
            hs[R + r] = b->h_pos[sl] + k;
            hs[2 * R + r] = tokens[r];
            hs[3 * R + r] = k;
        }
        b->h_pos[sl] += counts[i];
    }
    QIE_TRY(flush_table(b));
    hipStream_t st = e->stream;
    {   // the entries themselves (recurrent mixers walk an entry's rows in order) and their 16-row groups
        s->h_ent.clear();
        s->h_qgroups.clear();
        int row = 0;
        for (int i = 0; i < n_entries; i++) {
            const int p0 = b->h_pos[slots[i]] - counts[i];
            s->h_ent.push_back(int4{row, counts[i], slots[i], p0});
            for (int k = 0; k < counts[i]; k += 16) s->h_qgroups.push_back(int4{row + k, std::min(16, counts[i] - k), slots[i], p0 + k});
            row += counts[i];
        }
        if (n_entries > s->ent_cap || (int64_t)s->h_qgroups.size() > s->qgroups_cap) {
            QIE_HIP(hipStreamSynchronize(st));
            drop_graphs(s);
            if (s->d_ent) hipFree(s->d_ent);
            if (s->d_qgroups) hipFree(s->d_qgroups);
            s->d_ent = s->d_qgroups = nullptr;
            s->ent_cap = s->qgroups_cap = 0;
            const int64_t ce = std::max<int64_t>(b->B, n_entries), cg = ((int64_t)s->h_qgroups.size() + 255) / 256 * 256;
            QIE_TRY(dmalloc((void**)&s->d_ent, (size_t)ce * sizeof(int4)));
            QIE_TRY(dmalloc((void**)&s->d_qgroups, (size_t)cg * sizeof(int4)));
            s->ent_cap = ce;
            s->qgroups_cap = cg;
        }
        QIE_HIP(hipMemcpyAsync(s->d_ent, s->h_ent.data(), s->h_ent.size() * sizeof(int4), hipMemcpyHostToDevice, st));
        QIE_HIP(hipMemcpyAsync(s->d_qgroups, s->h_qgroups.data(), s->h_qgroups.size() * sizeof(int4), hipMemcpyHostToDevice, st));
        s->n_ent = n_entries;
        s->n_qgroups = (int)s->h_qgroups.size();
        s->max_count = 0;
        for (int i = 0; i < n_entries; i++) s->max_count = std::max(s->max_count, (int)counts[i]);
        if (s->slot_state > 0 && s->max_count > kScanLong) {
            s->h_chunks.clear();
            s->h_spans.clear();
            for (const int4& en : s->h_ent) {
                const int c0 = (int)s->h_chunks.size();
                for (int k = 0; k < en.y; k += kScanPiece)
                    s->h_chunks.push_back(int4{en.x + k, std::min(kScanPiece, en.y - k), (int)s->h_chunks.size(), 0});
                s->h_spans.push_back(int4{c0, (int)s->h_chunks.size() - c0, en.z, en.w});
            }
            const int64_t nc = (int64_t)s->h_chunks.size();
            if (nc > s->chunks_cap || nc > s->scan_cap) {
                QIE_HIP(hipStreamSynchronize(st));
                void* ps[] = {s->d_chunks, s->d_spans, s->s_loc, s->s_in, s->s_decay};
                for (void* q : ps)
                    if (q) hipFree(q);
                s->d_chunks = s->d_spans = nullptr;
                s->s_loc = s->s_in = s->s_decay = nullptr;
                s->chunks_cap = s->scan_cap = 0;
                const int64_t cap = (nc + 63) / 64 * 64;
                QIE_TRY(dmalloc((void**)&s->d_chunks, (size_t)cap * sizeof(int4)));
                QIE_TRY(dmalloc((void**)&s->d_spans, (size_t)std::max<int64_t>(b->B, n_entries) * sizeof(int4)));
                QIE_TRY(dmalloc((void**)&s->s_loc, (size_t)cap * s->m_state * 4));
                QIE_TRY(dmalloc((void**)&s->s_in, (size_t)cap * s->m_state * 4));
                QIE_TRY(dmalloc((void**)&s->s_decay, (size_t)cap * s->m_hd * 4));
                s->chunks_cap = s->scan_cap = cap;
            }
            QIE_HIP(hipMemcpyAsync(s->d_chunks, s->h_chunks.data(), s->h_chunks.size() * sizeof(int4), hipMemcpyHostToDevice, st));
            QIE_HIP(hipMemcpyAsync(s->d_spans, s->h_spans.data(), s->h_spans.size() * sizeof(int4), hipMemcpyHostToDevice, st));
            s->n_chunks = (int)nc;
        }
    }
    QIE_HIP(hipMemcpyAsync(s->row_slot, hs, (size_t)T * 4, hipMemcpyHostToDevice, st));
    QIE_HIP(hipMemcpyAsync(s->row_pos, hs + R, (size_t)T * 4, hipMemcpyHostToDevice, st));
    QIE_HIP(hipMemcpyAsync(s->tok, hs + 2 * R, (size_t)T * 4, hipMemcpyHostToDevice, st));
    QIE_HIP(hipMemcpyAsync(s->row_k, hs + 3 * R, (size_t)T * 4, hipMemcpyHostToDevice, st));
    QIE_TRY(build_groups(b, n_entries, counts));
    if (n_want > 0) QIE_HIP(hipMemcpyAsync(s->want, want_rows, (size_t)n_want * 4, hipMemcpyHostToDevice, st));
    QIE_TRY(run_forward(b, (int)T, n_want));
    s->last_T = (int)T;
    s->last_want = n_want;
    s->steps++;
    if (host_logits && n_want > 0)
        QIE_HIP(hipMemcpyAsync(host_logits, s->logits, (size_t)n_want * e->lm->a.vocab * 4, hipMemcpyDeviceToHost, st));
    // the staging rows and the caller's arrays are free again after this
    QIE_HIP(hipStreamSynchronize(st));
    return 0;
}

int qie_batch_step_sample(qie_batch* b, const qie_sampling* smp, int32_t* host_ids) {
    QIE_REQUIRE(b && b->lb && smp && host_ids, "qie_batch_step_sample: bad arguments");
    LayeredBatch* s = b->lb;
    const int n = s->last_want;
    QIE_REQUIRE(n > 0, "qie_batch_step_sample: the last step wanted no rows");
    qie_engine* e = b->e;
    hipStream_t st = e->stream;
    const int64_t V = e->lm->a.vocab;
    if (smp->top_k <= 1 || !(smp->temperature > 0.f)) {
        // greedy: on the fp32 rows themselves (two logits closer than a bf16 step stay apart)
        QIE_TRY(lay::argmax_rows(s->logits, n, V, s->d_ids, st));
    } else {
        QIE_TRY(lay::rows_to_bf16(s->logits, s->logits_bf, (int64_t)n * V, st));
        std::vector<int32_t> steps(n, (int32_t)(s->steps & 0x7fffffff));
        QIE_HIP(hipMemcpyAsync(s->d_step, steps.data(), (size_t)n * 4, hipMemcpyHostToDevice, st));
        QIE_HIP(hipStreamSynchronize(st));
        QIE_TRY(qie_sample(s->logits_bf, n, V, V, smp, s->d_step, s->d_ids, b->samp_ws, st));
    }
    QIE_HIP(hipMemcpyAsync(host_ids, s->d_ids, (size_t)n * 4, hipMemcpyDeviceToHost, st));
    QIE_HIP(hipStreamSynchronize(st));
    return 0;
}

int qie_batch_step_graphs(qie_batch* b, int32_t* n_graphs, int64_t* n_replays) {
    QIE_REQUIRE(b && b->lb, "qie_batch_step_graphs: a batch of a layered engine");
    int n = 0;
    for (const auto& g : b->lb->graphs) n += g.second.second != nullptr;
    if (n_graphs) *n_graphs = n;
    if (n_replays) *n_replays = b->lb->graph_replays;
    return 0;
}

int qie_engine_layer_runs(const qie_engine* e) { return e && e->lm ? (int)e->lm->runs.size() : 0; }

int qie_batch_keep_layers(qie_batch* b, int32_t enable) {
    QIE_REQUIRE(b && b->lb, "qie_batch_keep_layers: a batch of a layered engine");
    b->lb->keep_on = enable != 0;
    return 0;
}

int qie_batch_step_layers(qie_batch* b, float* host_out, int64_t n) {
    QIE_REQUIRE(b && b->lb && host_out, "qie_batch_step_layers: bad arguments");
    LayeredBatch* s = b->lb;
    const LayeredModel* m = b->e->lm;
    const int64_t W = m->a.width, T = s->last_T, L = (int64_t)m->runs.size();
    QIE_REQUIRE(s->keep && T > 0 && n >= L * T * W, "qie_batch_step_layers: nothing kept, or the buffer is too small");
    QIE_HIP(hipStreamSynchronize(b->e->stream));
    for (int64_t i = 0; i < L; i++)
        QIE_HIP(hipMemcpy(host_out + i * T * W, s->keep + i * s->cap * W, (size_t)T * W * 4, hipMemcpyDeviceToHost));
    return 0;
}

int qie_batch_time_stage(qie_batch* b, int32_t which, int32_t layer, int32_t iters, double* avg_us) {
    QIE_REQUIRE(b && b->lb && avg_us && iters > 0 && which >= 0 && which <= 4, "qie_batch_time_stage: bad arguments");
    LayeredBatch* s = b->lb;
    const LayeredModel* m = b->e->lm;
    const int T = s->last_T;
    QIE_REQUIRE(T > 0, "qie_batch_time_stage: run a step first");
    QIE_REQUIRE(which == 0 || (layer >= 0 && layer < m->a.n_layers), "qie_batch_time_stage: layer %d", layer);
    QIE_REQUIRE(which != 3 || m->L[layer].d.ff_kind != QIE_FF_NONE, "qie_batch_time_stage: layer %d has no feed-forward", layer);
    hipStream_t st = b->e->stream;
    hipEvent_t e0, e1;
    QIE_HIP(hipEventCreate(&e0));
    QIE_HIP(hipEventCreate(&e1));
    int rc = 0;
    const bool gqa = which != 0 && m->L[layer].d.mixer != QIE_MIXER_LATENT_ATTENTION;
    QIE_REQUIRE(which != 4 || m->L[layer].d.mixer == QIE_MIXER_GQA_RECURRENT || m->L[layer].d.mixer == QIE_MIXER_MINGRU ||
                    m->L[layer].d.mixer == QIE_MIXER_CHANNEL_DELTA,
                "qie_batch_time_stage: layer %d has no recurrence", layer);
    QIE_REQUIRE(which != 1 || (m->L[layer].d.mixer != QIE_MIXER_MINGRU && m->L[layer].d.mixer != QIE_MIXER_CHANNEL_DELTA),
                "qie_batch_time_stage: layer %d has no attention", layer);
    int run = 0;   // the layer's first run
    while (which != 0 && m->runs[run].layer != layer) run++;
    auto once = [&]() -> int {
        const float* xin = layer == 0 || which == 0 ? s->stack : s->x;
        if (gqa && m->L[layer].d.mixer == QIE_MIXER_CHANNEL_DELTA) {   // the slots' states are read, not advanced
            const LayerDev& L = m->L[layer];
            switch (which) {
                case 2:
                    QIE_TRY(enq_delta_proj(b, run, T));
                    return dense(b, s->ov, L.n_cat, L.wo, s->mix, m->a.width, T, m->a.width, L.n_cat, s->ov_bf);
                case 3: return enq_ff(b, layer, T);
                default: return enq_delta_scan(b, run, T, false);
            }
        }
        if (!gqa && which != 0 && m->a.block == QIE_BLOCK_PRENORM) {   // latent attention on the branch input s->y
            switch (which) {
                case 1: return enq_attention(b, layer, T);
                case 2:
                    QIE_TRY(enq_latent_proj(b, layer, T));
                    QIE_TRY(enq_absorb(b, layer, T));
                    return enq_mixer_out(b, layer, T);
                default: return enq_ff(b, layer, T);
            }
        }
        if (gqa) {   // the recurrence is timed from a zero state over the step's rows, the slots' states are not kept
            const LayerDev& L = m->L[layer];
            switch (which) {
                case 1: return enq_gqa_attention(b, run, T);
                case 2:
                    QIE_TRY(enq_gqa_proj(b, run, T));
                    return dense(b, s->ov, L.n_cat, L.wo, s->mix, m->a.width, T, m->a.width, L.n_cat, s->ov_bf);
                case 3: return enq_ff(b, layer, T);
                default: return L.d.mixer == QIE_MIXER_MINGRU ? enq_mingru(b, run, T) : enq_recurrence(b, run, T);
            }
        }
        switch (which) {
            case 0: return enq_forward(b, T, s->last_want);
            case 1: return enq_attention(b, layer, T);
            case 2:
                QIE_TRY(enq_input_proj(b, layer, xin, T, s->x_bf));
                QIE_TRY(enq_absorb(b, layer, T));
                return enq_mixer_out(b, layer, T);
            default: return enq_ff(b, layer, T);
        }
    };
    rc = once();   // warm
    if (!rc) {
        hipEventRecord(e0, st);
        for (int i = 0; i < iters && !rc; i++) rc = once();
        hipEventRecord(e1, st);
        hipError_t he = hipEventSynchronize(e1);
        float ms = 0.f;
        if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
        if (he != hipSuccess && !rc) rc = fail((int)he, "qie_batch_time_stage: %s", hipGetErrorString(he));
        *avg_us = (double)ms * 1000.0 / iters;
    }
    hipEventDestroy(e0);
    hipEventDestroy(e1);
    return rc;
}

}  // extern "C"
