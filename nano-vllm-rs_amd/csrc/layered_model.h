// layered_model.h — models described by their configuration file as a LIST OF LAYERS (the model registry, model_registry.cpp, maps an
// architecture name either to the dense Qwen3 graph of model_runner.cpp or to this family).  A layer is a token mixer — softmax attention
// over the paged K/V cache, or retention with a recurrent state — beside an optional feed-forward, both reading the same normalised
// residual stream; a range of layers can be run several times with the same weights, each pass with a cache / state of its own.
//
// The family shares the runner's step interface (sequences with a chunk [start, start + len) each: whole prompts, portions of prompts and
// single decoded tokens in one batch), the block manager's tables (K/V pages) and state slots (recurrent state, convolution history), the
// logits buffer and the samplers.
#pragma once
#include <hip/hip_runtime.h>
#include <map>
#include <string>
#include <vector>
#include "json.h"
#include "sequence.h"
#include "kernels/layered.h"

struct nvr_model_runner;

namespace nvr {

struct LayeredSpec {
    enum Mixer { ATTENTION = 0, RETENTION = 1 };
    struct Layer {
        int mixer = ATTENTION;
        int64_t heads = 0, kv_heads = 0, dim = 0, vdim = 0;
        double scale = 1.0;                                 // attention: score scale
        std::vector<double> decay;                          // retention: one per head
        int64_t rot_dims = 0; double rot_base = 10000.0;    // retention: rotated coordinates of q and k
        bool has_mlp = false; int64_t ff = 0; double limit = 0.0;
    };
    int64_t vocab = 0, width = 0;
    double embedding_scale = 1.0, eps = 1e-5, residual_mult = 1.0;
    int64_t taps = 1;                                       // causal convolution in front of every sublayer (1: a pointwise gain)
    std::vector<Layer> layers;
    std::vector<int> runs;                                  // layer index of every layer run, in order (loops unrolled)
    bool stateful() const { return true; }                  // convolution history, and recurrent state where there is retention
    static int parse_rugudra(const Json &cfg, LayeredSpec *out);   // (model_registry.cpp)
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
    };
    struct RunState { void *kc = nullptr, *vc = nullptr; float *state = nullptr, *hist = nullptr; };
    std::vector<LayerW> lw;
    std::vector<RunState> rs;
    void *embed = nullptr, *head = nullptr; float gfinal = 1.f;
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
                      std::vector<size_t> o_ftiles; std::vector<int32_t> n_ftiles; bool decode_sized; };
    int forward(nvr_model_runner &r, const StepPlan &p);
    int gemm(nvr_model_runner &r, const void *a, int64_t lda, const void *w, int64_t T, int64_t K, int64_t N, void *y, bool y_f32 = false);
    int put(nvr_model_runner &r, void *dst, int64_t dst_ld, int64_t rows, int64_t cols, int dtype, const void *src, bool as_operand);
};

}  // namespace nvr

// A parsed configuration file: which family runs it and that family's description (nvr_model_spec_from_json).
struct nvr_model_spec {
    std::string arch;
    int family = 0;                                         // 0: dense (nvr_model_config), 1: layered (LayeredSpec)
    nvr_model_config dense{};
    nvr::LayeredSpec layered;
};
