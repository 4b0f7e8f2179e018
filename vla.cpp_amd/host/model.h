// C++ engine API behind include/vla.h: the types and entry points of the
// reference's src/model.h:48-233 (Config, Inputs, Stats, model_load, predict,
// last_stats, config_is_sane) and the per-architecture base class of
// src/arch.h:83-103, restricted to what the action-expert attention path needs
// and extended with batched / phase-split calls.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

namespace vla {

struct Config {
    int64_t n_img = 0, n_lang = 0, n_state = 0, n_prefix = 0, n_suffix = 0, n_full = 0;
    int64_t hidden = 0, expert_h = 0, intermediate = 0, expert_inter = 0;
    int64_t n_q_heads = 0, n_kv_heads = 0, head_dim = 0, q_full_dim = 0, kv_full_dim = 0, n_layers = 0;
    int self_attn_every_n = 1;
    int64_t max_state_dim = 0, max_action_dim = 0, real_state_dim = 0, real_action_dim = 0;
    float norm_eps = 1e-8f;
    double min_period = 4e-3, max_period = 4.0;
    int num_steps = 10;
    float rms_eps = 1e-5f;
    int rope_n_dims = 0, rope_mode = 2;  // 2 = NeoX (GGML_ROPE_TYPE_NEOX)
    float rope_freq_base = 10000.f;
    bool denormalized = true;
};

enum class TimingDetail { NONE, PHASE };

struct Inputs {
    const float* precomputed_img_emb = nullptr;  // [n_img_views * n_img, hidden]
    int n_img_views = 0;
    const int32_t* lang_tokens = nullptr;
    int n_lang = 0;
    const float* state = nullptr;  // max_state_dim or null
    const float* noise = nullptr;  // n_actions * max_action_dim or null
    TimingDetail timing_detail = TimingDetail::NONE;
};

struct Stats {
    float ms_total = 0.f, ms_vision = 0.f, ms_inference = 0.f, ms_prefill = 0.f, ms_denoise = 0.f;
};

// One loaded architecture.  Holds mutable per-call state, so one call at a time
// per handle (the reference's rule, src/arch.h:85-87).
class ModelArch {
  public:
    virtual ~ModelArch();
    Config cfg;
    Stats stats;
    // Builds the prefix KV for `batch` observations and stages state / noise.
    virtual void prefill(const Inputs* in, int batch) = 0;
    // Runs `chunks` action chunks on `stream` without synchronising.
    void denoise(int chunks, void* stream) { denoise_steps(chunks * steps_per_chunk(), stream); }
    // Runs `n_steps` denoise steps (step index cycling through the chunk, the
    // noise re-staged at every chunk boundary) on `stream` without synchronising.
    // Whole chunks are replayed from a captured HIP graph once the shape has run
    // eagerly (set VLA_NO_GRAPH=1 to always launch eagerly).
    void denoise_steps(int n_steps, void* stream);
    virtual int steps_per_chunk() const = 0;

  protected:
    // Eager launches of steps [0, n_steps) of a chunk on `stream`.
    virtual void run_steps(int n_steps, void* stream) = 0;
    // Changes whenever anything baked into the launches changes (buffers, shapes, masks).
    virtual uint64_t launch_key() const = 0;

    // Per-launch timing for benchmarks.  While armed, prefill and run_steps record a HIP event
    // after every launch (prof_mark names what was launched since the previous mark) and
    // denoise launches eagerly instead of replaying its graph.
    void prof_start(const char* phase, void* stream);
    void prof_mark(const char* label);

  private:
    struct GraphState;
    GraphState* graph_ = nullptr;
    struct Profiler;
    Profiler* prof_ = nullptr;

  public:
    void drop_graph();
    // Arms the per-launch timing / synchronises, disarms and returns a JSON object
    // {"phase.label": {"us": average microseconds between the previous mark and this one,
    // "launches": marks recorded}, ...}.  The time between two marks is the launch's duration
    // plus the gap to its predecessor on the stream.
    void profile_begin();
    std::string profile_end();   // summary of the marks so far; the profiler stays armed
    void profile_discard();       // disarms and frees the marks
    // Synchronises and returns [batch, n_actions, max_action_dim].
    virtual std::vector<float> fetch() = 0;
    virtual int64_t n_actions() const = 0;
};

struct Model {
    ModelArch* arch = nullptr;
};

Model* model_load(const std::string& mmproj_path, const std::string& ckpt_path, const std::string& config_path = "");
void model_free(Model* m);
const Config& model_config(const Model* m);
std::vector<float> predict(Model* m, const Inputs& in);
const Stats& last_stats(const Model* m);
bool config_is_sane(const Config& c);

// CPU threads for host-side loaders, src/arch.h:43-53: VLA_N_THREADS or min(hw, 16).
int default_cpu_threads();

class Checkpoint;
ModelArch* flow_expert_create(const Checkpoint& ck);  // smolvla, pi0, gr00t_n1d5
ModelArch* bitvla_create(const Checkpoint& ck);

}  // namespace vla
