// layered_model.h — models described by their configuration file as a LIST OF LAYERS (the model registry, model_registry.cpp, maps an
// architecture name either to the dense Qwen3 graph of model_runner.cpp or to this family).  A layer is a token mixer and an optional feed-forward.
// Two layouts of a layer:
//   parallel (Rugudra)   — mixer and feed-forward read the same normalised residual stream (scalar-gain norm + short causal convolution); the mixer is softmax
//                          attention over paged K/V with a distance penalty and a sink, or retention; a range of layers can run several times with the same
//                          weights, each pass with a cache / state of its own;
//   sequential (Pusunex) — x <- x + nb(mixer(n(x))), then x <- x + nb(ff(n(x))) with RMS norms in groups before and after each sublayer; the mixer is latent
//                          attention (one cached latent row per token, optionally shared with an earlier layer, optionally with a rotated key part and a
//                          latent for the queries) or gated linear attention; the feed-forward is dense with a polynomial-norm activation or a mixture of
//                          experts; a per-layer token input and a weighted average over the outputs of all earlier layers close the layer.
//   scaled (Sosutar)     — x <- x + ls1 * mixer(n1(x)), then x <- x + ls2 * ff(n2(x)): RMS norms in front, a learned scale per channel behind each sublayer, learned
//                          positions added to the embedding; the mixer is an exponentially gated matrix memory (mLSTM), or a windowed attention (normed queries, keys
//                          and values, query temperature, linear distance penalty, sink, output gate) side by side with an elementwise gated recurrence (minGRU),
//                          each branch normed, half their sum; the feed-forward is dense with a squared ReLU; a layer may use an earlier layer's weights with a
//                          cache / state of its own.
//   joint (Sokalorn)     — x <- x + mixer(shift(n(x))) + ff(n(x)): ONE RMS norm per layer, read as it is by the feed-forward and through a token shift (a learned blend
//                          with the previous token's norm output) by the mixer; the mixer is a state-space layer (causal convolution, step sizes, a decay per head,
//                          input and output maps shared by groups of heads, gated group norm) or an attention without softmax (rotated queries and keys, capped scores,
//                          chunks of positions, sigmoid weights with a bias per head, output gate) side by side with a time-mixing recurrence (five shifted inputs, a
//                          decay per token and key channel, a bonus for the current token), each branch normed, half their sum; the feed-forward is a mixture of
//                          clamped gated experts (softmax router, renormalised top-k, a gated shared expert); a range of layers runs several times with the same
//                          weights, every pass starting with a product over [x ; embedding output] (layered_joint.cpp).
//
// The family shares the runner's step interface (sequences with a chunk [start, start + len) each: whole prompts, portions of prompts and
// single decoded tokens in one batch), the block manager's tables (K/V pages) and state slots (recurrent state, convolution history), the
// logits buffer and the samplers.
#pragma once
#include <hip/hip_runtime.h>
#include <map>
#include <string>
#include <vector>
#include "common.h"
#include "json.h"
#include "sequence.h"
#include "kernels/layered.h"

struct nvr_model_runner;

namespace nvr {

struct LayeredSpec {
    enum Mixer { ATTENTION = 0, RETENTION = 1, LATENT = 2, GLA = 3, MLSTM = 4, ATTN_GRU = 5, SSM = 6, ATTN_TMIX = 7 };
    enum Ff { FF_NONE = 0, FF_CLAMPED_GLU = 1, FF_POLY = 2, FF_MOE = 3, FF_RELU2 = 4, FF_MOE_GLU = 5 };
    enum Layout { PARALLEL = 0, SEQUENTIAL = 1, SCALED = 2, JOINT = 3 };
    struct Layer {
        int mixer = ATTENTION;
        int64_t heads = 0, kv_heads = 0, dim = 0, vdim = 0;
        double scale = 1.0;                                 // attention: score scale
        std::vector<double> decay;                          // retention: one per head
        int64_t rot_dims = 0; double rot_base = 10000.0;    // retention: rotated coordinates of q and k
        bool has_mlp = false; int64_t ff = 0; double limit = 0.0;
        // latent attention: size of the cached latent, of the queries' latent (0: queries straight from the layer's input), of the rotated key part shared by the
        // heads (0: none; rot_base its frequency base), the layer whose cached rows this layer reads (-1: its own), and whether sigmoid(W_g h) gates the heads' output
        int64_t kv_rank = 0, q_rank = 0, rot_dim = 0, kv_from = -1; bool out_gate = false;
        double tau = 1.0;                                   // gated linear attention: decay = sigmoid(z)^(1 / tau)
        double gate_cap = 0.0;                              // matrix memory: the log gates are cap * tanh(z / cap)
        int64_t window = 0;                                 // windowed attention: keys less than this many positions back (0: all)
        double temp_coef = 0.0; int64_t temp_every = 0;     // query temperature 1 + coef ln(floor((p + 1) / every) + 1) (every 0: none)
        int64_t gru_width = 0;                              // the gated recurrence beside the attention
        int64_t weights_of = -1;                            // the layer whose tensors this layer uses (-1: its own)
        int ff_kind = FF_NONE;
        int64_t experts = 0, top = 0, expert_ff = 0, shared_ff = 0;   // mixture of experts (shared_ff 0: no shared expert)
        double shared_limit = 0.0;                          // clamped gated experts: the shared expert's limit (the routed experts' is `limit`)
        // state-space mixer: heads x vdim channels, a state of dim x vdim per head, kv_heads groups of input / output maps; taps of its causal convolution and
        // the parts of its gated norm
        int64_t conv_taps = 1, mix_norm_groups = 1;
        // attention over chunks without softmax: position i sees j <= i with floor(j / chunk) == floor(i / chunk); scores capped at softcap (0: not); the rotation's
        // frequencies are divided by rot_factor
        int64_t chunk = 0; double softcap = 0.0, rot_factor = 1.0;
        int64_t t_heads = 0, t_dim = 0;                     // the time-mixing recurrence beside the attention: heads of t_dim x t_dim states
    };
    int layout = PARALLEL;
    int64_t norm_groups = 1;                                // sequential layout: RMS norms over this many equal parts of a row
    int64_t side_dim = 0;                                   // per-layer token input: numbers per layer and token (0: none)
    int64_t vocab = 0, width = 0;
    double embedding_scale = 1.0, eps = 1e-5, residual_mult = 1.0;
    int64_t max_positions = 0;                              // learned position vectors (0: none)
    double logit_scale = 1.0;
    int64_t taps = 1;                                       // causal convolution in front of every sublayer (1: a pointwise gain)
    std::vector<Layer> layers;
    std::vector<int> runs;                                  // layer index of every layer run, in order (loops unrolled)
    bool has_loop = false;                                  // joint layout: the configuration names a looped range (the checkpoint then holds its input product, used or not)
    std::vector<char> pass_start;                           // joint layout: this run starts a pass over the looped range (x <- W_loop [x ; embedding output] in front of it)
    bool stateful() const { return true; }                  // convolution history, and recurrent state where there is retention
    static int parse_rugudra(const Json &cfg, LayeredSpec *out);   // (model_registry.cpp)
    static int parse_pusunex(const Json &cfg, LayeredSpec *out);
    static int parse_sosutar(const Json &cfg, LayeredSpec *out);
    static int parse_sokalorn(const Json &cfg, LayeredSpec *out);
};

class LayeredModel {
public:
    LayeredSpec spec;
    bool bf16 = true;                                       // operand type: bfloat16 bits, or f32
    int64_t esz = 2;
    struct LayerW {
        void *mix = nullptr, *gu = nullptr, *out = nullptr; // [Nmix][W], [2 ff][W], [W][Kcat] (mixer output columns, then feed-forward columns)
        float *canon1 = nullptr, *canon2 = nullptr;         // [W][taps]
        float *r1 = nullptr, *r2 = nullptr, *sink = nullptr, *decay = nullptr, *freq = nullptr, *sin_t = nullptr;   // freq: the cosine table, sin_t: the sines ([positions][rot_dims / 2])
        float g1 = 1.f, g2 = 1.f;
        bool flash = false;                                 // attention prompts on the dense graph's flash kernel (penalty / sink form): row-major value pages
        float *pen = nullptr; bool pen_dirty = true;        // attention on the matrix cores: r1 * ln(1 + r2 * d) by head and distance
        int64_t nmix = 0, kcat = 0, mixcols = 0;            // rows of mix, columns of out, of which the mixer's
        int64_t qcol = 0, kcol = 0, vcol = 0, gcol = 0;
        // sequential layout
        float *n1 = nullptr, *n1b = nullptr, *n2 = nullptr, *n2b = nullptr;         // [W] each
        void *wx = nullptr;                                 // latent attention: [2 H Dv][kv_rank + R], keys (with identity rows for the rotated part) then values of all heads
        int64_t head_share = 0;                             // latent attention on the matrix cores: query heads per launch
        int64_t dcol = 0;                                   // latent attention: column of the (queries' latent,) cached row's source in the mix projection
        void *uq = nullptr, *ukt = nullptr, *uv = nullptr, *wo = nullptr;            // [H (D + R)][q_rank]; [H][kv_rank][D] (Wuk per head, transposed); [H][Dv][kv_rank]; [W][H Dv]
        float *dqn = nullptr, *dkvn = nullptr, *rfreq = nullptr;                     // latent norms' weights, rotation frequencies [rot_dim / 2]
        void *wa1 = nullptr, *wa2 = nullptr; int64_t a_rank = 0; float *a2b = nullptr, *hnorm = nullptr;   // gated linear attention: decay projections [a_rank][W], [H D][a_rank], bias, head norm [Dv]
        void *up = nullptr, *down = nullptr; float *act = nullptr;                   // dense feed-forward [ff][W], [W][ff]; 4 coefficients
        float *router = nullptr; void *egu = nullptr, *edown = nullptr, *sgu = nullptr, *sdown = nullptr;   // [E][W] f32; [E][2 f][W]; [E][W][f]; [2 fs][W]; [W][fs]
        void *sgate = nullptr, *sproj = nullptr; float *snorm = nullptr, *dwa = nullptr;   // [side][W], [W][side], [W]; [i + 2]
        // scaled layout (segments of mix start at multiples of 16 rows)
        float *ls1 = nullptr, *ls2 = nullptr;                                        // [W] each
        void *wgates = nullptr; int64_t gpad = 0; float *bi = nullptr, *bfg = nullptr;   // matrix memory: [gpad][W] (input gates' rows, then forget gates'), biases [H]
        float *qn = nullptr, *kn = nullptr, *slope = nullptr;                        // attention: norm weights over the whole q / k projection; distance slopes [H]
        int64_t zcol = 0, ucol = 0, rgcol = 0;                                       // gated recurrence: columns of z, x and its gate in the mix projection
        void *wo2 = nullptr; float *bz = nullptr, *bu = nullptr, *outl = nullptr, *outr = nullptr;   // [W][gru_width]; biases [gru_width]; the branches' norms [W]
        // joint layout
        float *shift = nullptr;                                                      // [W] token shift in front of the mixer
        float *convw = nullptr, *convb = nullptr, *dtb = nullptr, *alog = nullptr, *skip = nullptr;   // state-space mixer: [C][taps], [C], [H], [H], [H]
        int64_t ccol = 0, dtcol = 0, conv_c = 0;                                     // columns of the convolved channels and of the step sizes in the mix projection
        float *pb = nullptr; float *mu = nullptr;                                    // attention's bias per head; the five mixes' blends [5][W]
        void *w4 = nullptr, *w1 = nullptr, *w2 = nullptr; int64_t t_rank = 0;         // time mixing: r / k / v / g stacked [4][Ht Dt][W]; decay projections [rank][W], [Ht Dt][rank]
        float *w0 = nullptr, *bonus = nullptr, *tnorm = nullptr;                      // [Ht Dt] each
        void *router_op = nullptr;                                                   // [E + 1, padded to 16][W] operand type: the router's rows, then the shared expert's gate
    };
    struct RunState { void *kc = nullptr, *vc = nullptr; float *state = nullptr, *hist = nullptr; bool borrowed = false; void *rows = nullptr; float *mstate = nullptr;
                      float *shist = nullptr, *chist = nullptr; };   // joint layout: hist the norm output before the step [2][slots][W], shist the mixer input's (time mixing), chist the convolution's inputs   // mstate: a matrix memory's running maxima [slots][H]   // borrowed: another run's pages (a shared latent)
    std::vector<LayerW> lw;
    std::vector<RunState> rs;
    void *embed = nullptr, *head = nullptr; float gfinal = 1.f;
    // sequential layout
    float *wfinal = nullptr; void *side_embed = nullptr;                    // [W]; [vocab][layers * side_dim]
    float *kept = nullptr;                                                  // the embedding output and every layer's output: [layers + 1][max tokens][W] f32
    void *qlat = nullptr, *q2 = nullptr, *qabs = nullptr, *ctx = nullptr, *alow = nullptr, *az = nullptr, *act = nullptr, *shared_y = nullptr;
    bool flash_contiguous = false; void *kvx = nullptr;                      // flash tiles refer to rows of the step (not to block tables); expanded keys | values of a step
    int64_t alow_cap = 0; void *side_z = nullptr, *side_g = nullptr;
    // scaled layout
    void *pos = nullptr; void *tmp2 = nullptr, *gy = nullptr; float *gpre = nullptr, *tokg = nullptr, *gfloor = nullptr;   // [positions][W]; second branch's output, the recurrence's output; gates
    void *e_x = nullptr;                                                    // experts' inputs gathered in the order of the grouped rows
    void *e_gu = nullptr, *e_act = nullptr, *e_y = nullptr; int32_t *moe_i = nullptr; float *moe_score = nullptr;
    // joint layout
    void *loop_in = nullptr, *pair = nullptr; float *x0 = nullptr;          // [W][2 W]; [max tokens][2 W] operand rows; the embedding output
    void *conv_o = nullptr, *mixes = nullptr, *tproj = nullptr, *tlow = nullptr, *tz = nullptr, *tcat = nullptr; float *shared_g = nullptr;
    int64_t tlow_cap = 0; float *rlogits = nullptr;                          // router logits of a step [max tokens][experts + 1, padded]
    float *lm_part = nullptr;                          // arg-max partials of the 256 x 256 product with f32 output (not read)
    std::vector<void *> owned;                                              // device allocations of the sequential layout (freed with the model)
    // activations
    float *x = nullptr, *ret_o = nullptr;                                  // residual stream, retention outputs: f32
    void *proj = nullptr, *gu = nullptr, *tmp = nullptr, *a1 = nullptr, *a2 = nullptr, *cat = nullptr, *xsel = nullptr;   // operand type
    int64_t slots = 0; std::vector<int32_t> slot_par;
    std::vector<int64_t> flash_groups;                      // distinct H / G of the layers whose prompts take the flash kernel: one FlashTile list per value and step
    std::vector<int64_t> attn_groups;                       // distinct H / G of the attention layers: one list of query tiles per value and step
    void *attn_ws = nullptr; size_t attn_ws_bytes = 0;      // split-key partials of decode-sized steps
    // step inputs
    char *in_host = nullptr, *in_dev = nullptr; size_t in_bytes = 0;
    int64_t logit_rows_cap = 0;
    // decode-sized steps (one token per sequence) replay a captured hipGraph per (sequences, rows of logits, 256-token context bucket): the step's inputs
    // live at fixed places of the device arena, so a replay differs from its capture only in what the upload put there.  A key is captured the second
    // time it is seen (its first step also builds what is built once: penalty tables)
    std::map<uint64_t, hipGraphExec_t> graphs;
    uint64_t graph_replays = 0;

    ~LayeredModel();
    int init(nvr_model_runner &r);
    int execute(nvr_model_runner &r, nvr_seq *const *seqs, size_t nseq, const int32_t *want, size_t nwant);
    int load_tensor(nvr_model_runner &r, const char *name, int dtype, const int64_t *shape, int ndim, const void *data);

private:
    struct StepPlan { kl::Batch b; const int32_t *d_want; int64_t R, T, max_ctx; std::vector<size_t> o_tiles; std::vector<int32_t> n_tiles;
                      std::vector<size_t> o_ftiles; std::vector<int32_t> n_ftiles; bool decode_sized; bool whole_prompts = false; };
    int forward(nvr_model_runner &r, const StepPlan &p);
    int init_sequential(nvr_model_runner &r);
    int load_sequential(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data);
    int forward_sequential(nvr_model_runner &r, const StepPlan &p);
    int init_scaled(nvr_model_runner &r);
    int load_scaled(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data);
    int forward_scaled(nvr_model_runner &r, const StepPlan &p);
    int init_joint(nvr_model_runner &r);
    int load_joint(nvr_model_runner &r, const std::string &name, int dtype, const int64_t *shape, int ndim, const void *data);
    int forward_joint(nvr_model_runner &r, const StepPlan &p);
    template <class T> int own(T **p, size_t bytes);
    int gemm(nvr_model_runner &r, const void *a, int64_t lda, const void *w, int64_t T, int64_t K, int64_t N, void *y, bool y_f32 = false);
    int put(nvr_model_runner &r, void *dst, int64_t dst_ld, int64_t rows, int64_t cols, int dtype, const void *src, bool as_operand);
};

template <class T> int LayeredModel::own(T **p, size_t bytes) {            // zeroed device memory that lives as long as the model
    NVR_HIP_CHECK(hipMalloc((void **)p, bytes ? bytes : 16));
    owned.push_back((void *)*p);
    NVR_HIP_CHECK(hipMemset(*p, 0, bytes ? bytes : 16));
    return NVR_OK;
}

}  // namespace nvr

// A parsed configuration file: which family runs it and that family's description (nvr_model_spec_from_json).
struct nvr_model_spec {
    std::string arch;
    int family = 0;                                         // 0: dense (nvr_model_config), 1: layered (LayeredSpec)
    nvr_model_config dense{};
    nvr::LayeredSpec layered;
};
