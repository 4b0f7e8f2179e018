// Process-wide state of the kernel library: the tuning overrides (read from the
// environment once, never on a launch path) and the library's identification.

#include <stdlib.h>

#include <atomic>
#include <map>
#include <mutex>
#include <tuple>

#include "common.h"
#include "vla_kernels.h"

namespace vk {
namespace {

std::mutex g_mu;
Tuning g_tuning;
std::atomic<bool> g_loaded{false};
std::atomic<int> g_generation{0};  // bumped by every reload: holders of workspaces sized under the old overrides re-plan

int env_int(const char* name, int unset) {
    const char* e = getenv(name);
    return e ? atoi(e) : unset;
}

void load_locked() {
    Tuning t;
    t.attn_dl = env_int("VLA_ATTN_DL", -1);
    t.attn_slices = env_int("VLA_ATTN_SLICES", 0);
    t.attn_split_set = getenv("VLA_ATTN_SPLIT") != nullptr;
    t.attn_split = env_int("VLA_ATTN_SPLIT", -1);
    t.attn_part_f32 = getenv("VLA_ATTN_PART_F32") != nullptr;
    t.attn_no_arrive = getenv("VLA_ATTN_NO_ARRIVE") != nullptr;
    t.attn_no_direct = getenv("VLA_ATTN_NO_DIRECT") != nullptr;
    t.attn_no_stream = getenv("VLA_ATTN_NO_STREAM") != nullptr;
    t.gemm_rows_max = env_int("VLA_GEMM_ROWS_MAX", 32);
    t.attn_no_small = getenv("VLA_ATTN_NO_SMALL") != nullptr;
    t.attn_direct_rows = env_int("VLA_ATTN_DIRECT_ROWS", 32);
    t.gemm_tile = env_int("VLA_GEMM_TILE", -1);
    t.gemm_panel = env_int("VLA_GEMM_PANEL", 0);
    t.gemm_dl = env_int("VLA_GEMM_DL", -1);
    t.gemm_stages = env_int("VLA_GEMM_STAGES", 0);
    t.ternary_tile = env_int("VLA_TERNARY_TILE", 0);
    g_tuning = t;
    g_loaded.store(true, std::memory_order_release);
}

}  // namespace

const Tuning& tuning() {
    if (!g_loaded.load(std::memory_order_acquire)) {
        std::lock_guard<std::mutex> lk(g_mu);
        if (!g_loaded.load(std::memory_order_relaxed)) load_locked();
    }
    return g_tuning;
}

namespace {
struct Block {
    void* p = nullptr;
    size_t bytes = 0;
};
std::mutex g_scratch_mu;
std::map<std::tuple<int, int, hipStream_t>, Block> g_scratch;
}  // namespace

void* stream_scratch(int purpose, hipStream_t stream, size_t bytes) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    Block& b = g_scratch[std::make_tuple(purpose, dev, stream)];
    if (bytes <= b.bytes) return b.p;
    // the outgrown block is kept allocated: a captured graph may still hold its address
    size_t want = b.bytes ? b.bytes * 2 : (size_t)1 << 20;
    if (want < bytes) want = bytes;
    void* p = nullptr;
    if (hipMalloc(&p, want) != hipSuccess) return nullptr;
    if (hipMemset(p, 0, want) != hipSuccess) {
        (void)hipFree(p);
        return nullptr;
    }
    b.p = p;
    b.bytes = want;
    return p;
}

}  // namespace vk

extern "C" {

const char* vla_kernels_arch(void) { return "gfx950"; }

void vla_kernels_reload_env(void) {
    std::lock_guard<std::mutex> lk(vk::g_mu);
    vk::load_locked();
    vk::g_generation.fetch_add(1, std::memory_order_relaxed);
}

int vla_kernels_tuning_generation(void) { return vk::g_generation.load(std::memory_order_relaxed); }

}  // extern "C"
