// W8A8 "autotune" entry points of the reference API.
//
// On the RK3588 the tuner searches K/N tile sizes and A/C layout recipes for
// the NPU (reference src/rk_npu_quant_matmul.cpp:1144-1503).  None of those
// knobs changes what this build executes -- the HIP kernels pick their own
// tiling from the shape -- so every call returns ONE canonical strategy: the
// resources the reference would have fixed from the masks, a K partition that
// satisfies its conservative policy, its widest safe N tile and the plain
// layouts.  What IS measured is the strategy's latency: the blocking host API
// of this library is timed on seeded synthetic tensors with the caller's
// warm-up / loop / repeat counts, so `total_us` and `robust_us` mean what they
// mean in the reference.  The result cache keeps the reference's contract
// (value round trip, CACHE_MISS on any mismatch, atomic save, per-user default
// directory) in a small text format of its own.
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <chrono>
#include <cinttypes>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <set>
#include <string>
#include <vector>

#include "rk_host.h"
#include "rk_npu_quant_matmul.h"

namespace {

constexpr int kChannelTile = 32;   // N granularity of one NPU core (reference MIN_CHANNEL_TILE)
constexpr int kNTileSafeMax = 3072; // widest N tile the reference's tuner emits
constexpr int kKTileDefault = 2048; // its anchor K wave
constexpr const char* kMagic = "rk_npu_matmul_hip_tune";
constexpr int kFormat = 1;

int align_up_i(int v, int a) { return (v + a - 1) / a * a; }
int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

uint64_t affinity_mask() {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof(set), &set) != 0) return 1;
    uint64_t mask = 0;
    for (int c = 0; c < 64 && c < CPU_SETSIZE; ++c)
        if (CPU_ISSET(c, &set)) mask |= 1ull << c;
    return mask ? mask : 1;
}

// reference src/rk_npu_quant_matmul.cpp:75-81
bool valid_config(const rk_npu_matmul_autotune_config* c) {
    return c && c->M > 0 && c->N > 0 && c->K > 0 && (c->allowed_npu_core_mask & ~7u) == 0 && c->warmup >= 0 &&
           c->loops > 0 && c->repeats > 0 && c->timeout_ms > 0 && c->required_k_tile >= 0 &&
           c->required_k_tile <= c->K;
}

// reference :83-100
bool valid_family(const rk_npu_matmul_family_autotune_config* c) {
    if (!c || c->K <= 0 || c->N <= 0 || c->m_count <= 0 || !c->m_values || (c->allowed_npu_core_mask & ~7u) != 0 ||
        c->warmup < 0 || c->loops <= 0 || c->repeats <= 0 || c->timeout_ms == 0)
        return false;
    std::set<int> seen;
    for (int i = 0; i < c->m_count; ++i) {
        if (c->m_values[i] <= 0 || !seen.insert(c->m_values[i]).second) return false;
        if (c->frequencies && (!std::isfinite(c->frequencies[i]) || c->frequencies[i] <= 0)) return false;
    }
    return true;
}

bool valid_kind(int kind) { return kind >= RK_NPU_MATMUL_I8I8I32 && kind <= RK_NPU_MATMUL_F32I8F32_STATIC; }

// The reference keys its scores by execution backend (environment switches that
// move work between CPU and NPU); the switches do nothing here, but a cache
// written under one setting must still be refused under another
// (reference :136-146, :208).
uint32_t backend_mode(int kind) {
    auto on = [](const char* name) {
        const char* v = std::getenv(name);
        return v && std::strcmp(v, "1") == 0;
    };
    const bool dequant = kind != RK_NPU_MATMUL_I8I8I32 && on("RK_NPU_W8A8_NPU_DEQUANT");
    return ((on("RK_NPU_I8_NPU_REDUCE") || dequant) ? 1u : 0u) | (dequant ? 2u : 0u);
}

// Largest supported core set inside `allowed` with no more cores than N has
// 32-wide groups (reference src/rk_npu_autotune_common.cpp:57-63).
uint32_t pick_npu_mask(uint32_t allowed, int N) {
    const int groups = ceil_div_i(N, kChannelTile);
    for (uint32_t mask : {7u, 3u, 1u, 2u, 4u})
        if ((mask & allowed) == mask && __builtin_popcount(mask) <= groups) return mask;
    return 0;
}

// Up to four permitted CPUs, cores 4..7 first (reference :46-56).
uint64_t pick_cpu_mask(uint64_t allowed, int* count) {
    std::vector<int> order;
    for (int c = 4; c <= 7; ++c)
        if (allowed & (1ull << c)) order.push_back(c);
    for (int c = 0; c < 64; ++c)
        if ((c < 4 || c > 7) && (allowed & (1ull << c))) order.push_back(c);
    *count = std::min<int>(4, (int)order.size());
    uint64_t mask = 0;
    for (int i = 0; i < *count; ++i) mask |= 1ull << order[(size_t)i];
    return mask;
}

// reference src/rk_npu_quant_matmul.cpp:351-359
int pick_n_tile(int N, int groups) {
    const int align_n = std::max(kChannelTile, align_up_i(N, kChannelTile));
    int tile = align_up_i(ceil_div_i(align_n, groups), kChannelTile);
    if (ceil_div_i(align_n, tile) < groups)
        tile = std::max(kChannelTile, (align_n / groups / kChannelTile) * kChannelTile);
    return tile;
}

struct Key {
    int kind = 0, M = 0, N = 0, K = 0;
    uint32_t npu = 0;
    uint64_t cpu = 0;
    int warmup = 0, loops = 0, repeats = 0;
    uint32_t timeout = 0;
    int required_k_tile = 0;
    uint32_t mode = 0;
    bool operator==(const Key& o) const {
        return kind == o.kind && M == o.M && N == o.N && K == o.K && npu == o.npu && cpu == o.cpu &&
               warmup == o.warmup && loops == o.loops && repeats == o.repeats && timeout == o.timeout &&
               required_k_tile == o.required_k_tile && mode == o.mode;
    }
};

bool make_key(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* c, int kind, Key* key) {
    if (!ctx || !valid_config(c) || !valid_kind(kind)) return false;
    key->kind = kind;
    key->M = c->M;
    key->N = c->N;
    key->K = c->K;
    key->npu = c->allowed_npu_core_mask ? c->allowed_npu_core_mask : 7u;
    key->cpu = (c->allowed_cpu_core_mask ? c->allowed_cpu_core_mask : affinity_mask()) & affinity_mask();
    key->warmup = c->warmup;
    key->loops = c->loops;
    key->repeats = c->repeats;
    key->timeout = c->timeout_ms;
    key->required_k_tile = c->required_k_tile;
    key->mode = backend_mode(kind);
    return key->cpu != 0;
}

uint64_t key_hash(const Key& k) {
    uint64_t h = 0xcbf29ce484222325ull; // FNV-1a over the fields
    auto mix = [&](uint64_t v) {
        for (int i = 0; i < 8; ++i) {
            h ^= (v >> (8 * i)) & 0xff;
            h *= 0x100000001b3ull;
        }
    };
    mix(kFormat);
    mix((uint64_t)k.kind);
    mix((uint64_t)k.M);
    mix((uint64_t)k.N);
    mix((uint64_t)k.K);
    mix(k.npu);
    mix(k.cpu);
    mix((uint64_t)k.warmup);
    mix((uint64_t)k.loops);
    mix((uint64_t)k.repeats);
    mix(k.timeout);
    mix((uint64_t)k.required_k_tile);
    mix(k.mode);
    return h;
}

void print_strategy(FILE* f, const char* tag, const rk_npu_matmul_strategy& s) {
    std::fprintf(f, "%s %d %d %d %d %d %d %d %d %d %u %" PRIu64 " %d %.17g %.17g %.17g %.17g %.17g %.17g %.17g %d\n", tag,
                 (int)s.op_kind, s.M, s.N, s.K, s.k_tile, s.n_tile, (int)s.a_layout, s.wave_count, s.n_groups,
                 s.npu_core_mask, (uint64_t)s.cpu_core_mask, s.cpu_threads, s.input_us, s.npu_us, s.sync_us, s.output_us,
                 s.total_us, s.jitter_pct, s.robust_us, (int)s.c_layout);
}

bool scan_strategy(FILE* f, const char* tag, rk_npu_matmul_strategy* s) {
    char name[16] = {0};
    int kind = 0, a = 0, c = 0;
    uint64_t cpu = 0;
    std::memset(s, 0, sizeof(*s));
    const int n = std::fscanf(f, "%15s %d %d %d %d %d %d %d %d %d %u %" SCNu64 " %d %lf %lf %lf %lf %lf %lf %lf %d", name,
                              &kind, &s->M, &s->N, &s->K, &s->k_tile, &s->n_tile, &a, &s->wave_count, &s->n_groups,
                              &s->npu_core_mask, &cpu, &s->cpu_threads, &s->input_us, &s->npu_us, &s->sync_us,
                              &s->output_us, &s->total_us, &s->jitter_pct, &s->robust_us, &c);
    if (n != 21 || std::strcmp(name, tag) != 0) return false;
    s->op_kind = (rk_npu_matmul_op_kind)kind;
    s->a_layout = (rk_npu_matmul_a_layout)a;
    s->c_layout = (rk_npu_matmul_c_layout)c;
    s->cpu_core_mask = cpu;
    return true;
}

bool usable(const rk_npu_matmul_strategy& s, const Key& key) {
    rk_npu_matmul_workspace_requirements req;
    return (int)s.op_kind == key.kind && s.M == key.M && s.N == key.N && s.K == key.K &&
           (key.required_k_tile == 0 || s.k_tile == key.required_k_tile) && std::isfinite(s.total_us) &&
           s.total_us > 0 && rk_npu_matmul_workspace_memory_query(&s, &req) == RK_NPU_OK;
}

int cache_load(const char* path, const Key& key, rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable) {
    FILE* f = std::fopen(path, "r");
    if (!f) return RK_NPU_ERR_CACHE_MISS;
    char magic[40] = {0};
    int format = 0;
    Key got;
    uint64_t cpu = 0;
    bool ok = std::fscanf(f, "%39s %d", magic, &format) == 2 && std::strcmp(magic, kMagic) == 0 && format == kFormat;
    ok = ok && std::fscanf(f, " key %d %d %d %d %u %" SCNu64 " %d %d %d %u %d %u", &got.kind, &got.M, &got.N, &got.K,
                           &got.npu, &cpu, &got.warmup, &got.loops, &got.repeats, &got.timeout, &got.required_k_tile,
                           &got.mode) == 12;
    got.cpu = cpu;
    rk_npu_matmul_strategy a, b;
    ok = ok && got == key && scan_strategy(f, "fastest", &a) && scan_strategy(f, "stable", &b);
    std::fclose(f);
    if (!ok || !usable(a, key) || !usable(b, key)) return RK_NPU_ERR_CACHE_MISS;
    *fastest = a;
    *stable = b;
    return RK_NPU_OK;
}

int cache_save(const char* path, const Key& key, const rk_npu_matmul_strategy& fastest,
               const rk_npu_matmul_strategy& stable) {
    const std::string tmp = std::string(path) + ".tmp." + std::to_string((long long)getpid());
    FILE* f = std::fopen(tmp.c_str(), "w");
    if (!f) return RK_NPU_ERR_IO;
    std::fprintf(f, "%s %d\nkey %d %d %d %d %u %" PRIu64 " %d %d %d %u %d %u\n", kMagic, kFormat, key.kind, key.M, key.N,
                 key.K, key.npu, (uint64_t)key.cpu, key.warmup, key.loops, key.repeats, key.timeout, key.required_k_tile,
                 key.mode);
    print_strategy(f, "fastest", fastest);
    print_strategy(f, "stable", stable);
    const bool ok = std::fflush(f) == 0 && !std::ferror(f);
    std::fclose(f);
    if (!ok || std::rename(tmp.c_str(), path) != 0) {
        std::remove(tmp.c_str());
        return RK_NPU_ERR_IO;
    }
    return RK_NPU_OK;
}

bool make_dirs(const std::string& dir) {
    for (size_t i = 1; i <= dir.size(); ++i) {
        if (i == dir.size() || dir[i] == '/') {
            const std::string part = dir.substr(0, i);
            if (mkdir(part.c_str(), 0700) != 0 && errno != EEXIST) return false;
        }
    }
    return true;
}

// $XDG_CACHE_HOME/rk_npu_matmul or $HOME/.cache/rk_npu_matmul (reference header :243-245)
std::string default_directory() {
    const char* xdg = std::getenv("XDG_CACHE_HOME");
    if (xdg && *xdg) return std::string(xdg) + "/rk_npu_matmul";
    const char* home = std::getenv("HOME");
    return std::string(home && *home ? home : "/tmp") + "/.cache/rk_npu_matmul";
}

std::string file_in(const std::string& dir, const Key& key) {
    char name[40];
    std::snprintf(name, sizeof(name), "/%016" PRIx64 ".tune", key_hash(key));
    return dir + name;
}

// Deterministic tensors for timing (xorshift64*, fixed seed).
struct Rng {
    uint64_t s = 0x726b6e70755f6938ull;
    uint64_t next() {
        s ^= s >> 12;
        s ^= s << 25;
        s ^= s >> 27;
        return s * 0x2545f4914f6cdd1dull;
    }
};

uint16_t half_bits_of_small(float x) { // exact for the values generated below (multiples of 1/64 in [-2, 2])
    if (x == 0.0f) return 0;
    uint32_t u;
    std::memcpy(&u, &x, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int exp = (int)((u >> 23) & 0xff) - 127 + 15;
    return (uint16_t)(sign | ((uint32_t)exp << 10) | ((u & 0x7fffffu) >> 13));
}

// Time the blocking host API of the strategy; fills the timing fields.
int measure(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* c, rk_npu_matmul_strategy* s) {
    std::unique_ptr<rk_npu_iommu_domain, decltype(&rk_npu_iommu_domain_free)> domain(rk_npu_iommu_domain_create(ctx, 0),
                                                                                     rk_npu_iommu_domain_free);
    if (!domain) return RK_NPU_ERR_DOMAIN;
    const size_t M = (size_t)s->M, N = (size_t)s->N, K = (size_t)s->K;
    Rng rng;
    std::vector<int8_t> B(K * N);
    for (auto& v : B) v = (int8_t)((int)(rng.next() % 255) - 127);
    std::vector<float> w_scale(N), a_scale(M);
    for (auto& v : w_scale) v = 0.001f + (float)(rng.next() % 1000) * 1e-5f;
    for (auto& v : a_scale) v = 0.01f + (float)(rng.next() % 100) * 1e-4f;
    std::vector<float> Af(M * K);
    for (auto& v : Af) v = (float)((int)(rng.next() % 257) - 128) / 64.0f;
    const int kind = s->op_kind;
    const rk_npu_matmul_weight_config wc{s->K, s->N, s->k_tile};
    rk_npu_matmul_workspace* ws = rk_npu_matmul_workspace_create(domain.get(), s);
    if (!ws) return RK_NPU_ERR_NOMEM;
    int rc = RK_NPU_OK;
    std::vector<double> repeats;
    auto timed = [&](auto&& call) {
        for (int i = 0; i < c->warmup && rc == RK_NPU_OK; ++i) rc = call();
        for (int r = 0; r < c->repeats && rc == RK_NPU_OK; ++r) {
            const auto t0 = std::chrono::steady_clock::now();
            for (int i = 0; i < c->loops && rc == RK_NPU_OK; ++i) rc = call();
            const auto t1 = std::chrono::steady_clock::now();
            repeats.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count() / c->loops);
        }
    };
    if (kind == RK_NPU_MATMUL_I8I8I32) {
        std::vector<int8_t> A(M * K);
        for (auto& v : A) v = (int8_t)((int)(rng.next() % 255) - 127);
        std::vector<int32_t> Cout(M * N);
        rk_npu_i8i8i32_weights* w = rk_npu_i8i8i32_weights_create(domain.get(), &wc, B.data());
        if (!w) rc = RK_NPU_ERR_NOMEM;
        else timed([&] { return rk_npu_i8i8i32_run(ws, w, A.data(), Cout.data()); });
        rk_npu_i8i8i32_weights_free(w);
    } else if (kind == RK_NPU_MATMUL_F16I8F16_DYNAMIC || kind == RK_NPU_MATMUL_F16I8F16_STATIC) {
        std::vector<uint16_t> A(M * K), Cout(M * N);
        for (size_t i = 0; i < A.size(); ++i) A[i] = half_bits_of_small(Af[i]);
        rk_npu_f16i8f16_weights* w = rk_npu_f16i8f16_weights_create(domain.get(), &wc, B.data(), w_scale.data());
        if (!w) rc = RK_NPU_ERR_NOMEM;
        else if (kind == RK_NPU_MATMUL_F16I8F16_DYNAMIC)
            timed([&] { return rk_npu_f16i8f16_run_dynamic(ws, w, A.data(), Cout.data()); });
        else
            timed([&] { return rk_npu_f16i8f16_run_static(ws, w, A.data(), a_scale.data(), Cout.data()); });
        rk_npu_f16i8f16_weights_free(w);
    } else {
        std::vector<float> Cout(M * N);
        rk_npu_f32i8f32_weights* w = rk_npu_f32i8f32_weights_create(domain.get(), &wc, B.data(), w_scale.data());
        if (!w) rc = RK_NPU_ERR_NOMEM;
        else if (kind == RK_NPU_MATMUL_F32I8F32_DYNAMIC)
            timed([&] { return rk_npu_f32i8f32_run_dynamic(ws, w, Af.data(), Cout.data()); });
        else
            timed([&] { return rk_npu_f32i8f32_run_static(ws, w, Af.data(), a_scale.data(), Cout.data()); });
        rk_npu_f32i8f32_weights_free(w);
    }
    rk_npu_matmul_workspace_free(ws);
    if (rc != RK_NPU_OK) return rc;
    std::sort(repeats.begin(), repeats.end());
    const double median = repeats[repeats.size() / 2];
    const double spread = repeats.back() - repeats.front();
    s->total_us = median > 0 ? median : 1e-3;
    s->npu_us = s->total_us; // one fused device pass; the per-stage split of the reference does not exist here
    s->input_us = s->output_us = s->sync_us = 0;
    s->jitter_pct = s->total_us > 0 ? 100.0 * spread / s->total_us : 0;
    s->robust_us = s->total_us + 0.5 * spread; // reference src/rk_npu_autotune_common.cpp:36
    if (c->verbose)
        std::fprintf(stderr, "autotune: kind %d M %d N %d K %d Kt %d Nt %d -> %.2f us\n", kind, s->M, s->N, s->K, s->k_tile,
                     s->n_tile, s->total_us);
    return RK_NPU_OK;
}

int tune_one(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* c, int kind, rk_npu_matmul_strategy* fastest,
             rk_npu_matmul_strategy* stable) {
    if (!ctx || !valid_config(c) || !valid_kind(kind) || (!fastest && !stable)) return RK_NPU_ERR_PARAM;
    const uint32_t npu = pick_npu_mask(c->allowed_npu_core_mask ? c->allowed_npu_core_mask : 7u, c->N);
    int threads = 0;
    const uint64_t cpu =
        pick_cpu_mask((c->allowed_cpu_core_mask ? c->allowed_cpu_core_mask : affinity_mask()) & affinity_mask(), &threads);
    if (!npu || !threads) return RK_NPU_ERR_PARAM;
    const int k_tile = c->required_k_tile > 0 ? c->required_k_tile : std::min(c->K, kKTileDefault);
    if (rk_npu_matmul_k_partition_query(c->M, c->K, k_tile) != RK_NPU_OK) return RK_NPU_ERR_PARAM;
    const int cores = __builtin_popcount(npu);
    const int align_n = std::max(kChannelTile, align_up_i(c->N, kChannelTile));
    const int groups = std::max(cores, ceil_div_i(align_n, kNTileSafeMax));
    rk_npu_matmul_strategy s;
    std::memset(&s, 0, sizeof(s));
    s.op_kind = (rk_npu_matmul_op_kind)kind;
    s.M = c->M;
    s.N = c->N;
    s.K = c->K;
    s.k_tile = k_tile;
    s.n_tile = pick_n_tile(c->N, groups);
    s.a_layout = RK_NPU_MATMUL_A_LAYOUT_NORMAL;
    s.c_layout = RK_NPU_MATMUL_C_LAYOUT_NATIVE;
    s.wave_count = ceil_div_i(c->K, k_tile);
    s.n_groups = ceil_div_i(align_n, s.n_tile);
    s.npu_core_mask = npu;
    s.cpu_core_mask = cpu;
    s.cpu_threads = threads;
    const int rc = measure(ctx, c, &s);
    if (rc != RK_NPU_OK) return rc;
    if (fastest) *fastest = s;
    if (stable) *stable = s;
    return RK_NPU_OK;
}

int tune_cached(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* c, int kind, const char* cache_path, int refresh,
                rk_npu_matmul_strategy* fastest, rk_npu_matmul_strategy* stable, int* cache_hit) {
    if (cache_hit) *cache_hit = 0;
    Key key;
    if (!make_key(ctx, c, kind, &key) || (!fastest && !stable) || (cache_path && !*cache_path)) return RK_NPU_ERR_PARAM;
    std::string path;
    if (cache_path) {
        path = cache_path;
    } else {
        const std::string dir = default_directory();
        (void)make_dirs(dir);
        path = file_in(dir, key);
    }
    rk_npu_matmul_strategy a, b;
    if (!refresh && cache_load(path.c_str(), key, &a, &b) == RK_NPU_OK) {
        if (cache_hit) *cache_hit = 1;
    } else {
        const int rc = tune_one(ctx, c, kind, &a, &b);
        if (rc != RK_NPU_OK) return rc;
        (void)cache_save(path.c_str(), key, a, b); // a failed write never hides a good result
    }
    if (fastest) *fastest = a;
    if (stable) *stable = b;
    return RK_NPU_OK;
}

// One K partition for every M; per-M results optionally through the single-M cache.
int tune_family(rk_npu_ctx* ctx, const rk_npu_matmul_family_autotune_config* c, int kind, bool use_cache,
                const char* cache_directory, int refresh, rk_npu_matmul_family_summary* fast_summary,
                rk_npu_matmul_strategy* fast, rk_npu_matmul_family_summary* stable_summary,
                rk_npu_matmul_strategy* stable, int* hits, int* misses) {
    if (hits) *hits = 0;
    if (misses) *misses = 0;
    if (!ctx || !valid_family(c) || !valid_kind(kind) || (fast_summary == nullptr) != (fast == nullptr) ||
        (stable_summary == nullptr) != (stable == nullptr) || (!fast_summary && !stable_summary) ||
        (cache_directory && !*cache_directory))
        return RK_NPU_ERR_PARAM;
    const int k_tile = std::min(c->K, kKTileDefault);
    std::string dir;
    if (use_cache) {
        dir = cache_directory ? cache_directory : default_directory();
        if (!make_dirs(dir)) return RK_NPU_ERR_IO;
    }
    double weight_sum = 0, total = 0, robust = 0;
    for (int i = 0; i < c->m_count; ++i) {
        rk_npu_matmul_autotune_config one;
        std::memset(&one, 0, sizeof(one));
        one.M = c->m_values[i];
        one.N = c->N;
        one.K = c->K;
        one.allowed_npu_core_mask = c->allowed_npu_core_mask;
        one.allowed_cpu_core_mask = c->allowed_cpu_core_mask;
        one.warmup = c->warmup;
        one.loops = c->loops;
        one.repeats = c->repeats;
        one.timeout_ms = c->timeout_ms;
        one.verbose = c->verbose;
        one.required_k_tile = k_tile;
        rk_npu_matmul_strategy a, b;
        int rc;
        if (use_cache) {
            Key key;
            if (!make_key(ctx, &one, kind, &key)) return RK_NPU_ERR_PARAM;
            int hit = 0;
            rc = tune_cached(ctx, &one, kind, file_in(dir, key).c_str(), refresh, &a, &b, &hit);
            if (rc == RK_NPU_OK) {
                if (hits) *hits += hit;
                if (misses) *misses += !hit;
            }
        } else {
            rc = tune_one(ctx, &one, kind, &a, &b);
        }
        if (rc != RK_NPU_OK) return rc;
        const double f = c->frequencies ? c->frequencies[i] : 1.0;
        weight_sum += f;
        total += f * a.total_us;
        robust += f * b.robust_us;
        if (fast) fast[i] = a;
        if (stable) stable[i] = b;
    }
    const rk_npu_matmul_weight_config wc{c->K, c->N, k_tile};
    if (fast_summary) *fast_summary = {wc, total / weight_sum, robust / weight_sum};
    if (stable_summary) *stable_summary = {wc, total / weight_sum, robust / weight_sum};
    return RK_NPU_OK;
}

} // namespace

extern "C" {

// reference src/rk_npu_quant_matmul.cpp:1536-1550
void rk_npu_matmul_family_autotune_config_init(rk_npu_matmul_family_autotune_config* cfg, int N, int K, int m_count,
                                               const int* m_values) {
    if (!cfg) return;
    std::memset(cfg, 0, sizeof(*cfg));
    cfg->K = K;
    cfg->N = N;
    cfg->m_count = m_count;
    cfg->m_values = m_values;
    cfg->allowed_npu_core_mask = 7;
    cfg->warmup = 2;
    cfg->loops = 8;
    cfg->repeats = 3;
    cfg->timeout_ms = 500;
}

#define RK_TUNE_ENTRY(name, kind)                                                                            \
    int name(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg, rk_npu_matmul_strategy* fastest,     \
             rk_npu_matmul_strategy* stable) {                                                               \
        return tune_one(ctx, cfg, kind, fastest, stable);                                                    \
    }
RK_TUNE_ENTRY(rk_npu_i8i8i32_autotune, RK_NPU_MATMUL_I8I8I32)
RK_TUNE_ENTRY(rk_npu_f16i8f16_dynamic_autotune, RK_NPU_MATMUL_F16I8F16_DYNAMIC)
RK_TUNE_ENTRY(rk_npu_f16i8f16_static_autotune, RK_NPU_MATMUL_F16I8F16_STATIC)
RK_TUNE_ENTRY(rk_npu_f32i8f32_dynamic_autotune, RK_NPU_MATMUL_F32I8F32_DYNAMIC)
RK_TUNE_ENTRY(rk_npu_f32i8f32_static_autotune, RK_NPU_MATMUL_F32I8F32_STATIC)
#undef RK_TUNE_ENTRY

#define RK_FAMILY_ENTRY(name, kind)                                                                          \
    int name(rk_npu_ctx* ctx, const rk_npu_matmul_family_autotune_config* cfg,                               \
             rk_npu_matmul_family_summary* fastest_summary, rk_npu_matmul_strategy* fastest_strategies,      \
             rk_npu_matmul_family_summary* stable_summary, rk_npu_matmul_strategy* stable_strategies) {      \
        return tune_family(ctx, cfg, kind, false, nullptr, 0, fastest_summary, fastest_strategies,           \
                           stable_summary, stable_strategies, nullptr, nullptr);                             \
    }
RK_FAMILY_ENTRY(rk_npu_i8i8i32_autotune_family, RK_NPU_MATMUL_I8I8I32)
RK_FAMILY_ENTRY(rk_npu_f16i8f16_dynamic_autotune_family, RK_NPU_MATMUL_F16I8F16_DYNAMIC)
RK_FAMILY_ENTRY(rk_npu_f16i8f16_static_autotune_family, RK_NPU_MATMUL_F16I8F16_STATIC)
RK_FAMILY_ENTRY(rk_npu_f32i8f32_dynamic_autotune_family, RK_NPU_MATMUL_F32I8F32_DYNAMIC)
RK_FAMILY_ENTRY(rk_npu_f32i8f32_static_autotune_family, RK_NPU_MATMUL_F32I8F32_STATIC)
#undef RK_FAMILY_ENTRY

// reference src/rk_npu_quant_matmul.cpp:1552-1600
int rk_npu_matmul_autotune_cache_load(rk_npu_ctx* ctx, const char* cache_path, rk_npu_matmul_op_kind kind,
                                      const rk_npu_matmul_autotune_config* cfg, rk_npu_matmul_strategy* fastest,
                                      rk_npu_matmul_strategy* stable) {
    if (!cache_path || !*cache_path || !fastest || !stable) return RK_NPU_ERR_PARAM;
    Key key;
    if (!make_key(ctx, cfg, kind, &key)) return RK_NPU_ERR_PARAM;
    return cache_load(cache_path, key, fastest, stable);
}

int rk_npu_matmul_autotune_cache_save(rk_npu_ctx* ctx, const char* cache_path, rk_npu_matmul_op_kind kind,
                                      const rk_npu_matmul_autotune_config* cfg, const rk_npu_matmul_strategy* fastest,
                                      const rk_npu_matmul_strategy* stable) {
    if (!cache_path || !*cache_path || !fastest || !stable) return RK_NPU_ERR_PARAM;
    Key key;
    if (!make_key(ctx, cfg, kind, &key) || !usable(*fastest, key) || !usable(*stable, key)) return RK_NPU_ERR_PARAM;
    return cache_save(cache_path, key, *fastest, *stable);
}

int rk_npu_matmul_autotune_cached(rk_npu_ctx* ctx, const rk_npu_matmul_autotune_config* cfg, rk_npu_matmul_op_kind kind,
                                  const char* cache_path, int refresh, rk_npu_matmul_strategy* fastest,
                                  rk_npu_matmul_strategy* stable, int* cache_hit) {
    return tune_cached(ctx, cfg, kind, cache_path, refresh, fastest, stable, cache_hit);
}

int rk_npu_matmul_autotune_family_cached(rk_npu_ctx* ctx, const rk_npu_matmul_family_autotune_config* cfg,
                                         rk_npu_matmul_op_kind kind, const char* cache_directory, int refresh,
                                         rk_npu_matmul_family_summary* fastest_summary,
                                         rk_npu_matmul_strategy* fastest_strategies,
                                         rk_npu_matmul_family_summary* stable_summary,
                                         rk_npu_matmul_strategy* stable_strategies, int* cache_hits, int* cache_misses) {
    return tune_family(ctx, cfg, kind, true, cache_directory, refresh, fastest_summary, fastest_strategies, stable_summary,
                       stable_strategies, cache_hits, cache_misses);
}

// Weight constructors that quantize fp32 weights under a bits-per-weight budget
// for the NPU's lossless weight decompressor (reference :2009-2028): no such
// storage format exists here, so the budget search is reported as unmet.
rk_npu_f16i8f16_weights* rk_npu_f16i8f16_weights_create_from_f32_compress(rk_npu_iommu_domain*,
                                                                          const rk_npu_matmul_weight_config*,
                                                                          const float*, float) {
    errno = ENOTSUP;
    return nullptr;
}
rk_npu_f32i8f32_weights* rk_npu_f32i8f32_weights_create_from_f32_compress(rk_npu_iommu_domain*,
                                                                          const rk_npu_matmul_weight_config*,
                                                                          const float*, float) {
    errno = ENOTSUP;
    return nullptr;
}

} // extern "C"
