// Engine API: checkpoint loading, architecture dispatch and the one-shot
// predict() of src/model.cpp:200-296 over this library's architectures.

#include "model.h"

#include <algorithm>
#include <chrono>
#include <cstdlib>
#include <map>
#include <thread>

#include "checkpoint.h"
#include "device.h"

namespace vla {

int default_cpu_threads() {
    if (const char* e = std::getenv("VLA_N_THREADS")) {
        char* end = nullptr;
        const long n = std::strtol(e, &end, 10);
        if (end && *end == '\0' && n > 0 && n <= 1024) return (int)n;
        std::fprintf(stderr, "vla: ignoring VLA_N_THREADS='%s'\n", e);
    }
    const unsigned hw = std::thread::hardware_concurrency();
    return hw == 0 ? 4 : (int)std::min(hw, 16u);
}

// ---- whole-chunk HIP graph -------------------------------------------------
// A chunk is a fixed sequence of a few hundred short launches; replaying it as
// one graph removes the per-launch host cost that dominates at batch 1.  The
// graph holds kernel and device-to-device copy nodes only.
struct ModelArch::GraphState {
    hipStream_t cap_stream = nullptr;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    uint64_t key = 0;
    bool warmed = false;  // the shape has run eagerly once (lazy workspaces exist)
};

// ---- per-launch timing ------------------------------------------------------
struct ModelArch::Profiler {
    std::string phase;
    hipStream_t stream = nullptr;
    struct Mark {
        std::string label;  // empty: the opening event of a sequence
        hipEvent_t ev;
    };
    std::vector<Mark> marks;
    ~Profiler() {
        for (Mark& m : marks) (void)hipEventDestroy(m.ev);
    }
    void add(const std::string& label) {
        Mark m;
        m.label = label;
        VLA_HIP(hipEventCreate(&m.ev));
        VLA_HIP(hipEventRecord(m.ev, stream));
        marks.push_back(m);
    }
};

ModelArch::~ModelArch() {
    drop_graph();
    delete prof_;
}

void ModelArch::profile_begin() {
    delete prof_;
    prof_ = new Profiler();
}

void ModelArch::prof_start(const char* phase, void* stream) {
    if (!prof_) return;
    prof_->phase = phase;
    prof_->stream = (hipStream_t)stream;
    prof_->add("");
}

void ModelArch::prof_mark(const char* label) {
    if (!prof_) return;
    prof_->add(prof_->phase + "." + label);
}

void ModelArch::profile_discard() {
    delete prof_;
    prof_ = nullptr;
}

// The summary of the marks recorded so far.  The profiler stays armed: the caller disarms it
// (profile_discard) once the summary has been delivered, so a caller whose buffer was too
// small can come back with a larger one.
std::string ModelArch::profile_end() {
    if (!prof_) return "{}";
    VLA_HIP(hipDeviceSynchronize());
    std::map<std::string, std::pair<double, long>> acc;
    for (size_t i = 1; i < prof_->marks.size(); ++i) {
        if (prof_->marks[i].label.empty()) continue;
        float ms = 0.f;
        VLA_HIP(hipEventElapsedTime(&ms, prof_->marks[i - 1].ev, prof_->marks[i].ev));
        auto& a = acc[prof_->marks[i].label];
        a.first += (double)ms * 1e3;
        a.second += 1;
    }
    std::string out = "{";
    char buf[256];
    for (const auto& kv : acc) {
        std::snprintf(buf, sizeof(buf), "%s\"%s\": {\"us\": %.4f, \"launches\": %ld}", out.size() > 1 ? ", " : "", kv.first.c_str(),
                      kv.second.first / (double)kv.second.second, kv.second.second);
        out += buf;
    }
    return out + "}";
}

void ModelArch::drop_graph() {
    if (!graph_) return;
    if (graph_->exec) (void)hipGraphExecDestroy(graph_->exec);
    if (graph_->graph) (void)hipGraphDestroy(graph_->graph);
    if (graph_->cap_stream) (void)hipStreamDestroy(graph_->cap_stream);
    delete graph_;
    graph_ = nullptr;
}

void ModelArch::denoise_steps(int n_steps, void* stream) {
    static const bool no_graph = std::getenv("VLA_NO_GRAPH") != nullptr;
    const int spc = steps_per_chunk();
    int chunks = n_steps / spc;
    const int rem = n_steps % spc;
    hipStream_t st = (hipStream_t)stream;
    if (prof_) {  // timing every launch: eager, one sequence
        run_steps(n_steps, stream);
        return;
    }
    if (!graph_) graph_ = new GraphState();
    GraphState& g = *graph_;
    const uint64_t key = launch_key();
    if (g.key != key) {
        if (g.exec) (void)hipGraphExecDestroy(g.exec);
        if (g.graph) (void)hipGraphDestroy(g.graph);
        g.exec = nullptr;
        g.graph = nullptr;
        g.key = key;
        g.warmed = false;
    }
    while (chunks > 0) {
        if (no_graph || !g.warmed) {
            run_steps(spc, stream);
            g.warmed = true;
            --chunks;
            continue;
        }
        if (!g.exec) {
            if (!g.cap_stream) VLA_HIP(hipStreamCreateWithFlags(&g.cap_stream, hipStreamNonBlocking));
            VLA_HIP(hipStreamBeginCapture(g.cap_stream, hipStreamCaptureModeThreadLocal));
            try {
                run_steps(spc, g.cap_stream);
            } catch (...) {
                hipGraph_t junk = nullptr;
                (void)hipStreamEndCapture(g.cap_stream, &junk);
                if (junk) (void)hipGraphDestroy(junk);
                throw;
            }
            VLA_HIP(hipStreamEndCapture(g.cap_stream, &g.graph));
            VLA_HIP(hipGraphInstantiate(&g.exec, g.graph, nullptr, nullptr, 0));
        }
        VLA_HIP(hipGraphLaunch(g.exec, st));
        --chunks;
    }
    if (rem > 0) run_steps(rem, stream);
}

bool config_is_sane(const Config& c) {
    return c.real_action_dim <= c.max_action_dim && c.real_state_dim <= c.max_state_dim && c.real_action_dim >= 0 &&
           c.real_state_dim >= 0;
}

// ckpt_path: a GGUF written by the reference's converters (the tensors on the action-expert
// path are taken from it, gguf_import.cpp) or this library's VLAW container.
Model* model_load(const std::string&, const std::string& ckpt_path, const std::string&) {
    const Checkpoint ck = is_gguf_file(ckpt_path) ? import_gguf(ckpt_path) : Checkpoint(ckpt_path);
    const std::string arch = ck.str("arch");
    ModelArch* a = nullptr;
    if (arch == "smolvla" || arch == "pi0" || arch == "pi05" || arch == "gr00t_n1d5" || arch == "gr00t_n1d6") a = flow_expert_create(ck);
    else if (arch == "bitvla") a = bitvla_create(ck);
    else throw std::runtime_error("vla: unknown architecture '" + arch + "'");
    Model* m = new Model();
    m->arch = a;
    return m;
}

void model_free(Model* m) {
    if (!m) return;
    delete m->arch;
    delete m;
}

const Config& model_config(const Model* m) { return m->arch->cfg; }
const Stats& last_stats(const Model* m) { return m->arch->stats; }

std::vector<float> predict(Model* m, const Inputs& in) {
    using clk = std::chrono::steady_clock;
    const auto t0 = clk::now();
    ModelArch& a = *m->arch;
    a.stats = Stats{};
    a.prefill(&in, 1);
    const auto t1 = clk::now();
    a.denoise(1, nullptr);
    std::vector<float> out = a.fetch();
    const auto t2 = clk::now();
    const auto ms = [](clk::time_point x, clk::time_point y) { return std::chrono::duration<float, std::milli>(y - x).count(); };
    a.stats.ms_total = ms(t0, t2);
    a.stats.ms_inference = ms(t0, t2);
    if (in.timing_detail == TimingDetail::PHASE) {
        a.stats.ms_prefill = ms(t0, t1);
        a.stats.ms_denoise = ms(t1, t2);
    }
    return out;
}

}  // namespace vla
