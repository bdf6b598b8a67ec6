// W4A8 tuning entry points of the reference API (include/rk_npu_w4a8_tune.h).
//
// On the RK3588 the tuner times K/M/N tile sizes, CPU team sizes, serial /
// pipelined / chained submission and the panel8 input layout
// (reference src/rk_npu_w4a8_tune.cpp:31-118, src/rk_npu_w4a8_tune_policy.cpp:84-139).
// None of those knobs changes what this build executes, so every call returns
// ONE canonical strategy per shape: the resources the reference would have
// fixed from the masks, the widest K tile its weight-bound policy permits (or
// the required one), native input, CPU reduction, the full team, pipelined
// submission.  What IS real:
//  * the weight profile (INT16-partial certificate, multiplier policy,
//    fingerprint) -- it decides which K tiles are legal and ties a strategy
//    and a cache entry to one weight matrix;
//  * the timings -- the blocking host API of this library is run on the
//    reference's synthetic calibration tensor with the caller's warm-up / loop
//    / repeat counts, and its output is checked against a CPU restatement of
//    the operator before anything is reported;
//  * the cache contract (value round trip, CACHE_MISS on any mismatch, no
//    device work on a hit, atomic save), in a small text format of its own.
// A relaxed strategy (multiplier > 1) cannot overflow here: accumulation is
// int32, so the sample check that rejects a saturating tile on the NPU passes.
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cfloat>
#include <chrono>
#include <cinttypes>
#include <climits>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <new>
#include <set>
#include <string>
#include <vector>

#include "rk_host.h"
#include "rk_npu_w4a8_tune.h"
#include "rk_w4a8_internal.h"

using rkhost::W4Profile;

struct rk_npu_w4a8_tuning_profile {
    W4Profile value;
};

namespace {

constexpr uint32_t kRevision = 5;        // reference src/rk_npu_w4a8_tune_internal.h:13
constexpr int kSmallBatch = 8;           // reference :14
constexpr const char* kMagic = "rk_npu_w4a8_hip_tune";
constexpr int kFormat = 1;

using Strategy = rk_npu_w4a8_strategy_ex;

int align_up_i(int v, int a) { return (v + a - 1) / a * a; }
int ceil_div_i(int a, int b) { return (a + b - 1) / b; }

rk_npu_w4a8_options native_options() {
    return {(uint32_t)sizeof(rk_npu_w4a8_options), RK_NPU_W4A8_INPUT_NATIVE, RK_NPU_W4A8_REDUCE_CPU};
}
Strategy extend(const rk_npu_w4a8_strategy& s) { return {s, native_options()}; }
Strategy extend(const Strategy& s) { return s; }
void publish(rk_npu_w4a8_strategy* out, const Strategy& s) {
    if (out) *out = s.base;
}
void publish(Strategy* out, const Strategy& s) {
    if (out) *out = s;
}

uint64_t affinity_mask() {
    cpu_set_t set;
    CPU_ZERO(&set);
    if (sched_getaffinity(0, sizeof(set), &set) != 0) return 1;
    uint64_t mask = 0;
    for (int c = 0; c < 64 && c < CPU_SETSIZE; ++c)
        if (CPU_ISSET(c, &set)) mask |= 1ull << c;
    return mask ? mask : 1;
}

// ---- request, resource and strategy rules ---------------------------------------
// The rules themselves are API contract (reference src/rk_npu_w4a8_tune_policy.cpp:14-79,
// 140-164: which requests, schedules and cached strategies are acceptable); they are
// stated here as small predicates over named facts so that a rejected request can be
// traced to the rule that failed (RK_NPU_W4A8_TUNE_TRACE=1 prints it).

bool trace_rules() {
    static const bool on = [] {
        const char* v = std::getenv("RK_NPU_W4A8_TUNE_TRACE");
        return v && *v && *v != '0';
    }();
    return on;
}

struct Rule {
    const char* what;
    bool holds;
};
bool all_hold(const char* subject, std::initializer_list<Rule> rules) {
    for (const Rule& rule : rules)
        if (!rule.holds) {
            if (trace_rules()) std::fprintf(stderr, "[rk_npu_w4a8_tune] %s rejected: %s\n", subject, rule.what);
            return false;
        }
    return true;
}

// Row count up to which a problem may run chained: RK_NPU_W4A8_CHAIN_MAX_M, a decimal
// number 0..64; 8 when unset; -1 (nothing is valid) for anything else.
int chain_limit() {
    const char* text = std::getenv("RK_NPU_W4A8_CHAIN_MAX_M");
    if (!text) return 8;
    const size_t len = std::strlen(text);
    if (len == 0 || std::strspn(text, "0123456789") != len) return -1;
    const char* digits = text + std::strspn(text, "0"); // leading zeros carry no value
    if (std::strlen(digits) > 2) return -1;             // three significant digits exceed 64
    const int rows = *digits ? std::atoi(digits) : 0;
    return rows <= 64 ? rows : -1;
}

bool valid_config(const rk_npu_w4a8_autotune_config& c) {
    const int widest_tile = std::min(2048, align_up_i(std::max(c.K, 0), 32));
    const double mult = c.k_tile_multiplier;
    return all_hold("request", {
        {"1 <= M <= INT_MAX / 2", c.M >= 1 && c.M <= INT_MAX / 2},
        {"1 <= K <= INT32_MAX / 1024", c.K >= 1 && c.K <= INT32_MAX / 1024},
        {"1 <= N <= INT_MAX - 63", c.N >= 1 && c.N <= INT_MAX - 63},
        {"activations are fp32 or fp16", c.activation_type == RK_NPU_W4A8_F32 || c.activation_type == RK_NPU_W4A8_F16},
        {"NPU core mask within cores 0..2", (c.allowed_npu_core_mask & ~7u) == 0},
        {"warmup >= 0, loops >= 1, repeats >= 1", c.warmup >= 0 && c.loops >= 1 && c.repeats >= 1},
        {"timeout set", c.timeout_ms != 0},
        {"required K tile is 0 or a multiple of 32 up to min(2048, align32(K))",
         c.required_k_tile >= 0 && c.required_k_tile <= widest_tile && c.required_k_tile % 32 == 0},
        {"K tile multiplier is 0 (environment) or a finite number >= 1", std::isfinite(mult) && (mult == 0 || mult >= 1)},
    });
}

// Request checks, then the scan of the weights.
int make_profile(const rk_npu_w4a8_autotune_config& c, const int8_t* B, const float* w_scale, W4Profile* out) {
    if (!B || !w_scale || !valid_config(c)) return RK_NPU_ERR_PARAM;
    const double factor = c.k_tile_multiplier != 0 ? c.k_tile_multiplier : rkhost::w4a8_env_multiplier();
    if (factor < 1) return RK_NPU_ERR_PARAM; // malformed environment value
    W4Profile scanned;
    if (const int rc = rkhost::w4a8_make_profile(c.K, c.N, factor, B, w_scale, &scanned)) return rc;
    if (c.required_k_tile != 0 && !scanned.permits(c.required_k_tile)) return RK_NPU_ERR_PARAM;
    *out = scanned;
    return RK_NPU_OK;
}

// What a request is tuned on, fixed once from its masks and the process affinity: the NPU
// core set (the widest of {0,1,2}, {0,1}, {0}, {1}, {2} that the mask allows and that has
// no more cores than N has 64-column groups), and a team of up to four permitted CPUs,
// the RK3588's big cores 4..7 ahead of the others.
struct Resources {
    uint32_t npu = 0;
    uint64_t cpu = 0, allowed_cpu = 0;
    int threads = 0;
    int chain_max_m = 8;
};

uint32_t pick_npu_cores(uint32_t allowed, int N) {
    static const uint32_t kPreference[] = {7u, 3u, 1u, 2u, 4u};
    const int column_groups = ceil_div_i(N, 64);
    for (uint32_t set : kPreference)
        if ((allowed & set) == set && __builtin_popcount(set) <= column_groups) return set;
    return 0;
}

Resources make_resources(const rk_npu_w4a8_autotune_config& c) {
    Resources r;
    r.chain_max_m = chain_limit();
    if (r.chain_max_m < 0) return r;
    const uint64_t affinity = affinity_mask();
    r.allowed_cpu = affinity & (c.allowed_cpu_core_mask ? c.allowed_cpu_core_mask : affinity);
    const uint64_t big = r.allowed_cpu & 0xf0ull;
    for (uint64_t pool : {big, r.allowed_cpu & ~big}) // each pool in ascending CPU order
        while (pool && r.threads < 4) {
            const uint64_t lowest = pool & (~pool + 1);
            r.cpu |= lowest;
            pool ^= lowest;
            ++r.threads;
        }
    r.npu = pick_npu_cores(c.allowed_npu_core_mask ? c.allowed_npu_core_mask : 7u, c.N);
    return r;
}

// Which CPU team size and submission scheme a strategy may name, given the team the
// resources provide and the chaining limit.  Problems of few rows may also run on one
// thread and serially; chaining needs few enough rows and more than one K tile.
bool schedule_allowed(const rk_npu_w4a8_config& cfg, int team, int chain_rows) {
    if (team < 1 || team > 4 || chain_rows < 0) return false;
    const bool few_rows = cfg.M <= std::max(kSmallBatch, chain_rows);
    bool scheme_ok = false;
    switch (cfg.pipeline) {
    case RK_NPU_W4A8_PIPELINED: scheme_ok = true; break;
    case RK_NPU_W4A8_SERIAL: scheme_ok = few_rows; break;
    case RK_NPU_W4A8_CHAIN: scheme_ok = cfg.M <= chain_rows && cfg.k_tile < cfg.K; break;
    default: break;
    }
    const bool team_ok = cfg.cpu_threads == team || (few_rows && cfg.cpu_threads == 1);
    return team_ok && scheme_ok;
}

// A strategy taken on its own (tuned constructors, before any request is known).
bool valid_execution(const Strategy& s, bool panel8) {
    const rk_npu_w4a8_options& opt = s.execution;
    const bool layout_ok = opt.input_layout == RK_NPU_W4A8_INPUT_NATIVE ||
                           (panel8 && opt.input_layout == RK_NPU_W4A8_INPUT_PANEL8);
    if (!all_hold("strategy", {
            {"schedule fits its own CPU mask", schedule_allowed(s.base.config, __builtin_popcountll(s.base.cpu_core_mask), chain_limit())},
            {"options struct size", opt.struct_size == sizeof(opt)},
            {"CPU reduction", opt.reduce_backend == RK_NPU_W4A8_REDUCE_CPU},
            {"input layout", layout_ok},
        }))
        return false;
    rk_npu_w4a8_memory_info_ex unused{};
    return rk_npu_w4a8_memory_query_ex(&s.base.config, &opt, &unused) == RK_NPU_OK;
}

// A strategy against the request, weight profile and resources it claims to answer.
bool valid_strategy(const Strategy& strategy, const rk_npu_w4a8_autotune_config& c, const W4Profile& p,
                    const Resources& r, bool panel8) {
    if (!valid_execution(strategy, panel8)) return false;
    const rk_npu_w4a8_strategy& s = strategy.base;
    const rk_npu_w4a8_config& run = s.config;
    const rk_npu_w4a8_weight_info& wi = s.weights;
    static double rk_npu_w4a8_strategy::* const kTimes[] = {
        &rk_npu_w4a8_strategy::input_us, &rk_npu_w4a8_strategy::npu_us,     &rk_npu_w4a8_strategy::sync_us,
        &rk_npu_w4a8_strategy::output_us, &rk_npu_w4a8_strategy::total_us, &rk_npu_w4a8_strategy::jitter_pct,
        &rk_npu_w4a8_strategy::robust_us};
    bool times_ok = true;
    for (auto field : kTimes) times_ok = times_ok && std::isfinite(s.*field) && s.*field >= 0;
    return all_hold("strategy", {
        {"tuning revision", s.tuning_revision == kRevision},
        {"activation type", s.activation_type == c.activation_type},
        {"weight fingerprint", s.weight_fingerprint == p.fingerprint},
        {"shape", run.M == c.M && run.N == c.N && run.K == c.K},
        {"NPU core set", run.npu_core_mask == r.npu},
        {"CPU set", s.cpu_core_mask == r.cpu},
        {"schedule fits the resources", schedule_allowed(run, r.threads, r.chain_max_m)},
        {"timeout", run.timeout_ms == c.timeout_ms},
        {"K tile permitted by the weights", p.permits(run.k_tile)},
        {"K tile is the required one", c.required_k_tile == 0 || run.k_tile == c.required_k_tile},
        {"weight key", wi.config.K == c.K && wi.config.N == c.N && wi.config.k_tile == run.k_tile},
        {"weight bound", wi.safe_k_tile == p.safe && wi.multiplier == p.multiplier &&
                             wi.bound_relaxed == (p.certified(run.k_tile) ? 0 : 1)},
        {"timings finite and non-negative", times_ok},
    });
}

uint64_t double_bits(double d) {
    uint64_t u;
    std::memcpy(&u, &d, 8);
    return u;
}
double bits_double(uint64_t u) {
    double d;
    std::memcpy(&d, &u, 8);
    return d;
}

// Everything a cached result depends on, as one line of text
// (reference policy.cpp:165-175).
std::string make_key(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config& c, const W4Profile& p, const Resources& r,
                     bool panel8) {
    char text[512];
    std::snprintf(text, sizeof(text),
                  "%u %d %s %d %d %d %d %u %" PRIu64 " %u %" PRIu64 " %d %d %d %u %d %" PRIu64 " %d %" PRIu64
                  " %d %" PRIu64 " %d",
                  kRevision, panel8 ? 3 : 1, ctx->arch, c.M, c.N, c.K, (int)c.activation_type,
                  c.allowed_npu_core_mask ? c.allowed_npu_core_mask : 7u, (uint64_t)r.allowed_cpu, r.npu,
                  (uint64_t)r.cpu, c.warmup, c.loops, c.repeats, c.timeout_ms, c.required_k_tile, p.fingerprint, p.safe,
                  p.safe_tiles, p.limit, double_bits(p.multiplier), r.chain_max_m);
    return text;
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

// <directory or $XDG_CACHE_HOME/rk_npu_w4a8 or $HOME/.cache/rk_npu_w4a8>/<hash of the key>.tune
// (reference header: "NULL cache_path uses a separate rk_npu_w4a8 cache directory")
std::string cache_file(const std::string& key, const char* directory) {
    std::string dir;
    if (directory) {
        dir = directory;
    } else {
        const char* xdg = std::getenv("XDG_CACHE_HOME");
        const char* home = std::getenv("HOME");
        dir = xdg && *xdg ? std::string(xdg) + "/rk_npu_w4a8"
                          : std::string(home && *home ? home : "/tmp") + "/.cache/rk_npu_w4a8";
    }
    (void)make_dirs(dir);
    uint64_t h = 0xcbf29ce484222325ull;
    for (unsigned char ch : key) {
        h ^= ch;
        h *= 0x100000001b3ull;
    }
    char name[40];
    std::snprintf(name, sizeof(name), "/%016" PRIx64 ".tune", h);
    return dir + name;
}

void print_strategy(FILE* f, const char* tag, const Strategy& strategy) {
    const rk_npu_w4a8_strategy& s = strategy.base;
    const rk_npu_w4a8_config& c = s.config;
    const rk_npu_w4a8_weight_info& w = s.weights;
    std::fprintf(f, "%s %d %d %d %d %d %d %u %u %d %d %d %" PRIu64 " %d %d %d %d %" PRIu64 " %d %" PRIu64 " %u", tag, c.M,
                 c.N, c.K, c.m_tile, c.k_tile, c.n_tile, c.npu_core_mask, c.timeout_ms, c.pipeline, c.cpu_threads,
                 (int)s.activation_type, (uint64_t)s.cpu_core_mask, w.config.K, w.config.N, w.config.k_tile,
                 w.safe_k_tile, double_bits(w.multiplier), w.bound_relaxed, s.weight_fingerprint, s.tuning_revision);
    for (double d : {s.input_us, s.npu_us, s.sync_us, s.output_us, s.total_us, s.jitter_pct, s.robust_us})
        std::fprintf(f, " %" PRIu64, double_bits(d));
    std::fprintf(f, " %u %d %d\n", strategy.execution.struct_size, (int)strategy.execution.input_layout,
                 (int)strategy.execution.reduce_backend);
}

bool scan_strategy(FILE* f, const char* tag, Strategy* strategy) {
    *strategy = Strategy{};
    rk_npu_w4a8_strategy& s = strategy->base;
    rk_npu_w4a8_config& c = s.config;
    rk_npu_w4a8_weight_info& w = s.weights;
    char name[16] = {0};
    int dtype = 0, layout = 0, reduce = 0;
    uint64_t cpu = 0, factor = 0, fingerprint = 0, times[7] = {0};
    const int n = std::fscanf(f,
                              "%15s %d %d %d %d %d %d %u %u %d %d %d %" SCNu64 " %d %d %d %d %" SCNu64 " %d %" SCNu64
                              " %u %" SCNu64 " %" SCNu64 " %" SCNu64 " %" SCNu64 " %" SCNu64 " %" SCNu64 " %" SCNu64
                              " %u %d %d",
                              name, &c.M, &c.N, &c.K, &c.m_tile, &c.k_tile, &c.n_tile, &c.npu_core_mask, &c.timeout_ms,
                              &c.pipeline, &c.cpu_threads, &dtype, &cpu, &w.config.K, &w.config.N, &w.config.k_tile,
                              &w.safe_k_tile, &factor, &w.bound_relaxed, &fingerprint, &s.tuning_revision, &times[0],
                              &times[1], &times[2], &times[3], &times[4], &times[5], &times[6],
                              &strategy->execution.struct_size, &layout, &reduce);
    if (n != 31 || std::strcmp(name, tag) != 0 || (dtype != RK_NPU_W4A8_F32 && dtype != RK_NPU_W4A8_F16) ||
        (layout != RK_NPU_W4A8_INPUT_NATIVE && layout != RK_NPU_W4A8_INPUT_PANEL8) || reduce != RK_NPU_W4A8_REDUCE_CPU)
        return false;
    s.activation_type = (rk_npu_w4a8_activation_type)dtype;
    s.cpu_core_mask = cpu;
    w.multiplier = bits_double(factor);
    s.weight_fingerprint = fingerprint;
    double* fields[7] = {&s.input_us, &s.npu_us, &s.sync_us, &s.output_us, &s.total_us, &s.jitter_pct, &s.robust_us};
    for (int i = 0; i < 7; ++i) *fields[i] = bits_double(times[i]);
    strategy->execution.input_layout = (rk_npu_w4a8_input_layout)layout;
    strategy->execution.reduce_backend = (rk_npu_w4a8_reduce_backend)reduce;
    return true;
}

int cache_load(const std::string& path, const std::string& key, const rk_npu_w4a8_autotune_config& c,
               const W4Profile& p, const Resources& r, Strategy* fast, Strategy* stable, bool panel8) {
    FILE* f = std::fopen(path.c_str(), "r");
    if (!f) return RK_NPU_ERR_CACHE_MISS;
    char magic[40] = {0};
    int format = 0;
    std::vector<char> line(key.size() + 8);
    bool ok = std::fscanf(f, "%39s %d\n", magic, &format) == 2 && std::strcmp(magic, kMagic) == 0 && format == kFormat;
    ok = ok && std::fgets(line.data(), (int)line.size(), f) != nullptr;
    if (ok) {
        std::string got(line.data());
        while (!got.empty() && (got.back() == '\n' || got.back() == '\r')) got.pop_back();
        ok = got == key;
    }
    Strategy a, b;
    ok = ok && scan_strategy(f, "fastest", &a) && scan_strategy(f, "stable", &b);
    std::fclose(f);
    if (!ok || !valid_strategy(a, c, p, r, panel8) || !valid_strategy(b, c, p, r, panel8)) return RK_NPU_ERR_CACHE_MISS;
    *fast = a;
    *stable = b;
    return RK_NPU_OK;
}

int cache_save(const std::string& path, const std::string& key, const Strategy& fast, const Strategy& stable) {
    const std::string tmp = path + ".tmp." + std::to_string((long long)getpid());
    FILE* f = std::fopen(tmp.c_str(), "w");
    if (!f) return RK_NPU_ERR_IO;
    std::fprintf(f, "%s %d\n%s\n", kMagic, kFormat, key.c_str());
    print_strategy(f, "fastest", fast);
    print_strategy(f, "stable", stable);
    const bool ok = std::fflush(f) == 0 && !std::ferror(f);
    std::fclose(f);
    if (!ok || std::rename(tmp.c_str(), path.c_str()) != 0) {
        std::remove(tmp.c_str());
        return RK_NPU_ERR_IO;
    }
    return RK_NPU_OK;
}

// IEEE binary16 bits of a value that is exactly representable (the calibration
// values below are multiples of 1/32 of magnitude < 4).
uint16_t exact_half_bits(float x) {
    if (x == 0.0f) return 0;
    uint32_t u;
    std::memcpy(&u, &x, 4);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const int exp = (int)((u >> 23) & 0xff) - 127 + 15;
    return (uint16_t)(sign | ((uint32_t)exp << 10) | ((u & 0x7fffffu) >> 13));
}

// float -> binary16, round to nearest even (for checking fp16 outputs).
uint16_t half_bits_rne(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t abs = x & 0x7fffffffu;
    if (abs >= 0x7f800000u) return (uint16_t)(sign | 0x7c00u | (abs > 0x7f800000u ? 0x200u | ((abs >> 13) & 0x3ffu) : 0));
    if (abs >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u); // rounds to infinity
    if (abs < 0x33000001u) return (uint16_t)sign;              // rounds to zero
    int exp = (int)(abs >> 23) - 127;
    uint32_t mant = (abs & 0x7fffffu) | 0x800000u;
    int shift = 13;
    if (exp < -14) {
        shift += -14 - exp;
        exp = -15;
    }
    const uint32_t kept = mant >> shift, rest = mant & ((1u << shift) - 1), halfway = 1u << (shift - 1);
    uint32_t h = ((uint32_t)(exp + 15) << 10) + (kept & (exp == -15 ? 0xffffffffu : 0x3ffu));
    if (exp == -15) h = kept;
    if (rest > halfway || (rest == halfway && (kept & 1))) ++h;
    return (uint16_t)(sign | h);
}

// The calibration tensor and the output check of a tuning run
// (reference src/rk_npu_w4a8_tune_data.cpp:8-48): a fixed LCG fills A with
// multiples of 1/32 (an all-zero first row when M >= 3), and the operator's
// result must equal  (float(sum_k q*B) * a_scale) * w_scale  bit for bit, on
// every column when the problem is small and on 17 evenly spaced columns
// otherwise.
struct Calibration {
    int M, K, N;
    bool half;
    std::vector<float> a, c;
    std::vector<uint16_t> ah, ch;
    explicit Calibration(const rk_npu_w4a8_autotune_config& cfg)
        : M(cfg.M), K(cfg.K), N(cfg.N), half(cfg.activation_type == RK_NPU_W4A8_F16), a((size_t)M * K),
          c((size_t)M * N) {
        if (half) {
            ah.resize(a.size());
            ch.resize(c.size());
        }
        uint32_t state = 0x57344138u;
        for (size_t i = 0; i < a.size(); ++i) {
            state = state * 1664525u + 1013904223u;
            const bool zero_row = M >= 3 && i < (size_t)K;
            a[i] = zero_row ? 0.0f : (float)((int)((state >> 16) % 255) - 127) * 0.03125f;
            if (half) ah[i] = exact_half_bits(a[i]);
        }
    }
    int run(rk_npu_w4a8_workspace* ws, const rk_npu_w4a8_weights* w, rk_npu_w4a8_timings* t) {
        return half ? rk_npu_w4a8_run_f16(ws, w, ah.data(), ch.data(), t) : rk_npu_w4a8_run_f32(ws, w, a.data(), c.data(), t);
    }
    bool output_correct(const int8_t* B, const float* w_scale) const {
        std::vector<int> columns;
        if ((int64_t)M * K <= 16000000 / (int64_t)N) {
            for (int n = 0; n < N; ++n) columns.push_back(n);
        } else {
            for (int i = 0; i < 17; ++i) columns.push_back((int)((int64_t)i * (N - 1) / 16));
        }
        std::vector<int8_t> q((size_t)K);
        for (int m = 0; m < M; ++m) {
            const float* row = a.data() + (size_t)m * K;
            float maximum = 0;
            for (int k = 0; k < K; ++k) maximum = std::max(maximum, std::fabs(row[k]));
            const float scale = maximum == 0 ? 1.0f : std::max(maximum / 127.0f, FLT_MIN), inv = 1.0f / scale;
            for (int k = 0; k < K; ++k)
                q[(size_t)k] = (int8_t)std::min(127.0f, std::max(-127.0f, std::round(row[k] * inv)));
            for (int n : columns) {
                int64_t sum = 0;
                for (int k = 0; k < K; ++k) sum += (int)q[(size_t)k] * (int)B[(size_t)k * N + n];
                const float partial = (float)sum * scale;
                const float expected = partial * w_scale[n];
                const size_t i = (size_t)m * N + n;
                if (half ? ch[i] != half_bits_rne(expected) : std::memcmp(&c[i], &expected, 4) != 0) return false;
            }
        }
        return true;
    }
};

double median_of(std::vector<double> v) {
    std::sort(v.begin(), v.end());
    return v[v.size() / 2];
}

// One tuning run: builds the canonical strategy, checks its output, times it.
int tune_one(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config& c, const int8_t* B, const float* w_scale,
             const W4Profile& p, const Resources& r, Strategy* fast, Strategy* stable) {
    const int k_tile = c.required_k_tile ? c.required_k_tile : p.limit;
    if (!p.permits(k_tile)) return RK_NPU_ERR_PARAM;
    const int cores = __builtin_popcount(r.npu);
    const int max_shard = ceil_div_i(ceil_div_i(c.N, 64), cores) * 64;
    Strategy s{};
    s.execution = native_options();
    rk_npu_w4a8_config& cfg = s.base.config;
    cfg = {c.M, c.N, c.K, std::min(64, c.M), k_tile, std::min(1024, max_shard), r.npu, c.timeout_ms,
           RK_NPU_W4A8_PIPELINED, r.threads};
    rk_npu_w4a8_memory_info_ex memory{};
    if (rk_npu_w4a8_memory_query_ex(&cfg, &s.execution, &memory) != RK_NPU_OK) return RK_NPU_ERR_PARAM;

    std::unique_ptr<rk_npu_iommu_domain, decltype(&rk_npu_iommu_domain_free)> domain(rk_npu_iommu_domain_create(ctx, 0),
                                                                                     rk_npu_iommu_domain_free);
    if (!domain) return RK_NPU_ERR_DOMAIN;
    std::unique_ptr<rk_npu_w4a8_weights, decltype(&rk_npu_w4a8_weights_free)> w(
        rkhost::w4a8_create_weights(domain.get(), p.info(k_tile), B, w_scale, &p), rk_npu_w4a8_weights_free);
    std::unique_ptr<rk_npu_w4a8_workspace, decltype(&rk_npu_w4a8_workspace_free)> ws(
        rk_npu_w4a8_workspace_create_ex(domain.get(), &cfg, &s.execution), rk_npu_w4a8_workspace_free);
    if (!w || !ws) return RK_NPU_ERR_NOMEM;

    Calibration data(c);
    rk_npu_w4a8_timings t{};
    int rc = data.run(ws.get(), w.get(), &t);
    if (rc) return rc;
    if (!data.output_correct(B, w_scale)) return RK_NPU_ERR_PARAM;
    for (int i = 0; i < c.warmup && !rc; ++i) rc = data.run(ws.get(), w.get(), &t);
    std::vector<double> input, device, sync, output, total;
    for (int rep = 0; rep < c.repeats && !rc; ++rep) {
        double in = 0, dev = 0, sy = 0, out = 0;
        const auto t0 = std::chrono::steady_clock::now();
        for (int i = 0; i < c.loops && !rc; ++i) {
            rc = data.run(ws.get(), w.get(), &t);
            in += t.activation_scan_us + t.quant_pack_us;
            dev += t.submit_us;
            sy += t.sync_us;
            out += t.reduce_us + t.dequant_us;
        }
        const auto t1 = std::chrono::steady_clock::now();
        total.push_back(std::chrono::duration<double, std::micro>(t1 - t0).count() / c.loops);
        input.push_back(in / c.loops);
        device.push_back(dev / c.loops);
        sync.push_back(sy / c.loops);
        output.push_back(out / c.loops);
    }
    if (rc) return rc;
    rk_npu_w4a8_strategy& b = s.base;
    b.activation_type = c.activation_type;
    b.cpu_core_mask = r.cpu;
    b.weights = p.info(k_tile);
    b.weight_fingerprint = p.fingerprint;
    b.tuning_revision = kRevision;
    b.input_us = median_of(input);
    b.npu_us = median_of(device);
    b.sync_us = median_of(sync);
    b.output_us = median_of(output);
    b.total_us = std::max(median_of(total), 1e-3);
    const double spread = *std::max_element(total.begin(), total.end()) - *std::min_element(total.begin(), total.end());
    b.jitter_pct = 100.0 * spread / b.total_us;
    b.robust_us = b.total_us + 0.5 * spread; // reference src/rk_npu_autotune_common.cpp:36
    if (c.verbose)
        std::fprintf(stderr, "w4 autotune: M/K/N=%d/%d/%d k_tile=%d total=%.2f robust=%.2f us relaxed=%d\n", c.M, c.K, c.N,
                     k_tile, b.total_us, b.robust_us, b.weights.bound_relaxed);
    *fast = s;
    *stable = s;
    return RK_NPU_OK;
}

int tune_cached(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config& c, const int8_t* B, const float* w_scale,
                const W4Profile& p, const Resources& r, const std::string& file, const std::string& key, int refresh,
                Strategy* fast, Strategy* stable, int* hit, bool panel8) {
    if (hit) *hit = 0;
    if (!refresh && cache_load(file, key, c, p, r, fast, stable, panel8) == RK_NPU_OK) {
        if (hit) *hit = 1;
        return RK_NPU_OK;
    }
    const int rc = tune_one(ctx, c, B, w_scale, p, r, fast, stable);
    if (rc) return rc;
    const int saved = cache_save(file, key, *fast, *stable); // a failed write never hides a good result
    if (saved && c.verbose) std::fprintf(stderr, "w4 autotune: cache save failed (%d), strategy remains valid\n", saved);
    return RK_NPU_OK;
}

// reference src/rk_npu_w4a8_tune.cpp:120-142
template <class S>
int entry(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B, const float* w_scale,
          const char* path, int refresh, S* fast, S* stable, int* hit, bool cache) {
    constexpr bool panel8 = std::is_same<S, Strategy>::value;
    if (hit) *hit = 0;
    if (!ctx || !c || (!fast && !stable) || (path && !*path)) return RK_NPU_ERR_PARAM;
    try {
        W4Profile p;
        int rc = make_profile(*c, B, w_scale, &p);
        if (rc) return rc;
        const Resources r = make_resources(*c);
        if (!r.npu || !r.threads) return RK_NPU_ERR_PARAM;
        Strategy f{}, s{};
        if (cache) {
            const std::string key = make_key(ctx, *c, p, r, panel8);
            rc = tune_cached(ctx, *c, B, w_scale, p, r, path ? std::string(path) : cache_file(key, nullptr), key,
                             refresh, &f, &s, hit, panel8);
        } else {
            rc = tune_one(ctx, *c, B, w_scale, p, r, &f, &s);
        }
        if (!rc) {
            publish(fast, f);
            publish(stable, s);
        }
        return rc;
    } catch (const std::bad_alloc&) {
        return RK_NPU_ERR_NOMEM;
    } catch (...) {
        return RK_NPU_ERR_PARAM;
    }
}

// reference src/rk_npu_w4a8_tune_cache.cpp:68-98
template <class S>
int load_entry(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B, const float* w_scale,
               const char* path, S* fast, S* stable) {
    constexpr bool panel8 = std::is_same<S, Strategy>::value;
    if (!ctx || !c || !fast || !stable || (path && !*path)) return RK_NPU_ERR_PARAM;
    try {
        W4Profile p;
        int rc = make_profile(*c, B, w_scale, &p);
        if (rc) return rc;
        const Resources r = make_resources(*c);
        if (!r.npu || !r.threads) return RK_NPU_ERR_PARAM;
        const std::string key = make_key(ctx, *c, p, r, panel8);
        Strategy f{}, s{};
        rc = cache_load(path ? std::string(path) : cache_file(key, nullptr), key, *c, p, r, &f, &s, panel8);
        if (!rc) {
            publish(fast, f);
            publish(stable, s);
        }
        return rc;
    } catch (const std::bad_alloc&) {
        return RK_NPU_ERR_NOMEM;
    } catch (...) {
        return RK_NPU_ERR_PARAM;
    }
}

template <class S>
int save_entry(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B, const float* w_scale,
               const char* path, const S* fast, const S* stable) {
    constexpr bool panel8 = std::is_same<S, Strategy>::value;
    if (!ctx || !c || !fast || !stable || (path && !*path)) return RK_NPU_ERR_PARAM;
    try {
        W4Profile p;
        const int rc = make_profile(*c, B, w_scale, &p);
        if (rc) return rc;
        const Resources r = make_resources(*c);
        if (!r.npu || !r.threads) return RK_NPU_ERR_PARAM;
        const Strategy f = extend(*fast), s = extend(*stable);
        if (!valid_strategy(f, *c, p, r, panel8) || !valid_strategy(s, *c, p, r, panel8)) return RK_NPU_ERR_PARAM;
        const std::string key = make_key(ctx, *c, p, r, panel8);
        return cache_save(path ? std::string(path) : cache_file(key, nullptr), key, f, s);
    } catch (const std::bad_alloc&) {
        return RK_NPU_ERR_NOMEM;
    } catch (...) {
        return RK_NPU_ERR_PARAM;
    }
}

// reference src/rk_npu_w4a8_tune_policy.cpp:186-204
rk_npu_w4a8_weights* create_tuned(rk_npu_iommu_domain* domain, const Strategy& strategy, const int8_t* B,
                                  const float* w_scale, bool panel8) {
    const rk_npu_w4a8_strategy& s = strategy.base;
    if (!domain || !B || !w_scale) return nullptr;
    try {
        rk_npu_w4a8_autotune_config c;
        rk_npu_w4a8_autotune_config_init(&c, s.config.M, s.config.N, s.config.K);
        c.activation_type = s.activation_type;
        c.required_k_tile = s.config.k_tile;
        c.k_tile_multiplier = s.weights.multiplier;
        c.timeout_ms = s.config.timeout_ms;
        W4Profile p;
        if (make_profile(c, B, w_scale, &p)) return nullptr;
        const Resources r{s.config.npu_core_mask, s.cpu_core_mask, s.cpu_core_mask, __builtin_popcountll(s.cpu_core_mask),
                          chain_limit()};
        if (!valid_strategy(strategy, c, p, r, panel8)) return nullptr;
        return rkhost::w4a8_create_weights(domain, p.info(c.required_k_tile), B, w_scale, &p);
    } catch (...) {
        return nullptr;
    }
}

// A family shares ONE K partition over all its M values.  The reference times
// each of its K-tile candidates for every M and keeps the tile with the best
// frequency-weighted time (src/rk_npu_w4a8_tune_family.cpp:31-55); every tile
// runs the same kernels here, so the family takes the tile a single-M call
// would take (the required one, else the widest permitted) and measures each M
// once -- through the single-M cache entries when caching, which is what lets
// a later run with more M values, or other frequencies, reuse them.
template <class S>
int family(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* cfg, const int8_t* B, const float* w_scale,
           const char* directory, int refresh, rk_npu_w4a8_family_summary* fast, S* fs,
           rk_npu_w4a8_family_summary* stable, S* ss, int* hits, int* misses, bool cache) {
    constexpr bool panel8 = std::is_same<S, Strategy>::value;
    if (hits) *hits = 0;
    if (misses) *misses = 0;
    if (!ctx || !cfg || cfg->m_count < 1 || !cfg->m_values || (!fast && !stable) || bool(fast) != bool(fs) ||
        bool(stable) != bool(ss) || (directory && !*directory))
        return RK_NPU_ERR_PARAM;
    try {
        const size_t count = (size_t)cfg->m_count;
        std::vector<double> share(count);
        std::set<int> seen;
        double total_weight = 0;
        for (size_t i = 0; i < count; ++i) {
            const int m = cfg->m_values[i];
            share[i] = cfg->frequencies ? cfg->frequencies[i] : 1.0;
            if (m < 1 || m > INT_MAX / 2 || !seen.insert(m).second || !std::isfinite(share[i]) || share[i] <= 0)
                return RK_NPU_ERR_PARAM;
            total_weight += share[i];
        }
        if (!std::isfinite(total_weight)) return RK_NPU_ERR_PARAM;
        for (double& f : share) f /= total_weight;

        rk_npu_w4a8_autotune_config one = cfg->base;
        one.M = 1;
        W4Profile p;
        int rc = make_profile(one, B, w_scale, &p);
        if (rc) return rc;
        const Resources r = make_resources(one);
        if (!r.npu || !r.threads) return RK_NPU_ERR_PARAM;
        one.required_k_tile = one.required_k_tile ? one.required_k_tile : p.limit;

        std::vector<Strategy> f(count), s(count);
        int hit_count = 0, miss_count = 0;
        for (size_t i = 0; i < count; ++i) {
            one.M = cfg->m_values[i];
            if (cache) {
                const std::string key = make_key(ctx, one, p, r, panel8);
                int hit = 0;
                rc = tune_cached(ctx, one, B, w_scale, p, r, cache_file(key, directory), key, refresh, &f[i], &s[i],
                                 &hit, panel8);
                hit_count += !rc && hit;
                miss_count += !rc && !hit;
            } else {
                rc = tune_one(ctx, one, B, w_scale, p, r, &f[i], &s[i]);
            }
            if (rc) break;
        }
        if (hits) *hits = hit_count;
        if (misses) *misses = miss_count;
        if (rc) return rc;
        auto report = [&](rk_npu_w4a8_family_summary* summary, S* out, const std::vector<Strategy>& chosen) {
            if (!summary) return;
            *summary = {chosen[0].base.weights, p.fingerprint, 0, 0};
            for (size_t i = 0; i < count; ++i) {
                publish(out + i, chosen[i]);
                summary->weighted_total_us += share[i] * chosen[i].base.total_us;
                summary->weighted_robust_us += share[i] * chosen[i].base.robust_us;
            }
        };
        report(fast, fs, f);
        report(stable, ss, s);
        return RK_NPU_OK;
    } catch (const std::bad_alloc&) {
        return RK_NPU_ERR_NOMEM;
    } catch (...) {
        return RK_NPU_ERR_PARAM;
    }
}

} // namespace

extern "C" {

// reference src/rk_npu_w4a8_tune_policy.cpp:178-185
void rk_npu_w4a8_autotune_config_init(rk_npu_w4a8_autotune_config* c, int M, int N, int K) {
    if (c) *c = {M, N, K, RK_NPU_W4A8_F32, 7, 0, 2, 8, 3, 500, 0, 0, 0};
}
void rk_npu_w4a8_family_config_init(rk_npu_w4a8_family_config* c, int N, int K, int m_count, const int* m_values) {
    if (!c) return;
    *c = {};
    rk_npu_w4a8_autotune_config_init(&c->base, 1, N, K);
    c->m_count = m_count;
    c->m_values = m_values;
}

// reference src/rk_npu_w4a8.cpp:287-295
rk_npu_w4a8_tuning_profile* rk_npu_w4a8_tuning_profile_from_weights(const rk_npu_w4a8_weights* weights) {
    if (!weights) return nullptr;
    return new (std::nothrow) rk_npu_w4a8_tuning_profile{rkhost::w4a8_profile_of(weights)};
}
void rk_npu_w4a8_tuning_profile_free(rk_npu_w4a8_tuning_profile* profile) { delete profile; }
uint64_t rk_npu_w4a8_tuning_profile_fingerprint(const rk_npu_w4a8_tuning_profile* profile) {
    return profile ? profile->value.fingerprint : 0;
}

int rk_npu_w4a8_autotune(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B, const float* w_scale,
                         rk_npu_w4a8_strategy* fastest, rk_npu_w4a8_strategy* stable) {
    return entry(ctx, c, B, w_scale, nullptr, 0, fastest, stable, nullptr, false);
}
int rk_npu_w4a8_autotune_cached(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                const float* w_scale, const char* cache_path, int refresh,
                                rk_npu_w4a8_strategy* fastest, rk_npu_w4a8_strategy* stable, int* cache_hit) {
    return entry(ctx, c, B, w_scale, cache_path, refresh, fastest, stable, cache_hit, true);
}
int rk_npu_w4a8_autotune_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                            const float* w_scale, rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable) {
    return entry(ctx, c, B, w_scale, nullptr, 0, fastest, stable, nullptr, false);
}
int rk_npu_w4a8_autotune_cached_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                   const float* w_scale, const char* cache_path, int refresh,
                                   rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable, int* cache_hit) {
    return entry(ctx, c, B, w_scale, cache_path, refresh, fastest, stable, cache_hit, true);
}

int rk_npu_w4a8_autotune_cache_load(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                    const float* w_scale, const char* cache_path, rk_npu_w4a8_strategy* fastest,
                                    rk_npu_w4a8_strategy* stable) {
    return load_entry(ctx, c, B, w_scale, cache_path, fastest, stable);
}
int rk_npu_w4a8_autotune_cache_save(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                    const float* w_scale, const char* cache_path, const rk_npu_w4a8_strategy* fastest,
                                    const rk_npu_w4a8_strategy* stable) {
    return save_entry(ctx, c, B, w_scale, cache_path, fastest, stable);
}
int rk_npu_w4a8_autotune_cache_load_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                       const float* w_scale, const char* cache_path, rk_npu_w4a8_strategy_ex* fastest,
                                       rk_npu_w4a8_strategy_ex* stable) {
    return load_entry(ctx, c, B, w_scale, cache_path, fastest, stable);
}
int rk_npu_w4a8_autotune_cache_save_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c, const int8_t* B,
                                       const float* w_scale, const char* cache_path,
                                       const rk_npu_w4a8_strategy_ex* fastest, const rk_npu_w4a8_strategy_ex* stable) {
    return save_entry(ctx, c, B, w_scale, cache_path, fastest, stable);
}

// reference src/rk_npu_w4a8_tune_cache.cpp:107-121: no weight scan, no device
// work; the captured profile must carry the SAME explicit multiplier.
int rk_npu_w4a8_autotune_cache_load_profile_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_autotune_config* c,
                                               const rk_npu_w4a8_tuning_profile* profile, const char* cache_path,
                                               rk_npu_w4a8_strategy_ex* fastest, rk_npu_w4a8_strategy_ex* stable) {
    if (!ctx || !c || !profile || !fastest || !stable || (cache_path && !*cache_path) || !valid_config(*c))
        return RK_NPU_ERR_PARAM;
    try {
        const W4Profile& p = profile->value;
        if (p.K != c->K || p.N != c->N || c->k_tile_multiplier != p.multiplier ||
            (c->required_k_tile && !p.permits(c->required_k_tile)))
            return RK_NPU_ERR_PARAM;
        const Resources r = make_resources(*c);
        if (!r.npu || !r.threads) return RK_NPU_ERR_PARAM;
        const std::string key = make_key(ctx, *c, p, r, true);
        return cache_load(cache_path ? std::string(cache_path) : cache_file(key, nullptr), key, *c, p, r, fastest,
                          stable, true);
    } catch (const std::bad_alloc&) {
        return RK_NPU_ERR_NOMEM;
    } catch (...) {
        return RK_NPU_ERR_PARAM;
    }
}

rk_npu_w4a8_weights* rk_npu_w4a8_weights_create_tuned(rk_npu_iommu_domain* domain, const rk_npu_w4a8_strategy* s,
                                                      const int8_t* B, const float* w_scale) {
    return s ? create_tuned(domain, extend(*s), B, w_scale, false) : nullptr;
}
rk_npu_w4a8_weights* rk_npu_w4a8_weights_create_tuned_ex(rk_npu_iommu_domain* domain,
                                                         const rk_npu_w4a8_strategy_ex* s, const int8_t* B,
                                                         const float* w_scale) {
    return s ? create_tuned(domain, *s, B, w_scale, true) : nullptr;
}
// reference src/rk_npu_w4a8_tune_policy.cpp:205-212
rk_npu_w4a8_workspace* rk_npu_w4a8_workspace_create_tuned_ex(rk_npu_iommu_domain* domain,
                                                             const rk_npu_w4a8_strategy_ex* s) {
    if (!s || s->base.tuning_revision != kRevision || !valid_execution(*s, true) ||
        s->base.config.K != s->base.weights.config.K || s->base.config.N != s->base.weights.config.N ||
        s->base.config.k_tile != s->base.weights.config.k_tile)
        return nullptr;
    return rk_npu_w4a8_workspace_create_ex(domain, &s->base.config, &s->execution);
}

int rk_npu_w4a8_autotune_family(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* c, const int8_t* B,
                                const float* w_scale, rk_npu_w4a8_family_summary* fastest,
                                rk_npu_w4a8_strategy* fastest_strategies, rk_npu_w4a8_family_summary* stable,
                                rk_npu_w4a8_strategy* stable_strategies) {
    return family(ctx, c, B, w_scale, nullptr, 0, fastest, fastest_strategies, stable, stable_strategies, nullptr,
                  nullptr, false);
}
int rk_npu_w4a8_autotune_family_cached(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* c, const int8_t* B,
                                       const float* w_scale, const char* cache_directory, int refresh,
                                       rk_npu_w4a8_family_summary* fastest, rk_npu_w4a8_strategy* fastest_strategies,
                                       rk_npu_w4a8_family_summary* stable, rk_npu_w4a8_strategy* stable_strategies,
                                       int* cache_hits, int* cache_misses) {
    return family(ctx, c, B, w_scale, cache_directory, refresh, fastest, fastest_strategies, stable, stable_strategies,
                  cache_hits, cache_misses, true);
}
int rk_npu_w4a8_autotune_family_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* c, const int8_t* B,
                                   const float* w_scale, rk_npu_w4a8_family_summary* fastest,
                                   rk_npu_w4a8_strategy_ex* fastest_strategies, rk_npu_w4a8_family_summary* stable,
                                   rk_npu_w4a8_strategy_ex* stable_strategies) {
    return family(ctx, c, B, w_scale, nullptr, 0, fastest, fastest_strategies, stable, stable_strategies, nullptr,
                  nullptr, false);
}
int rk_npu_w4a8_autotune_family_cached_ex(rk_npu_ctx* ctx, const rk_npu_w4a8_family_config* c, const int8_t* B,
                                          const float* w_scale, const char* cache_directory, int refresh,
                                          rk_npu_w4a8_family_summary* fastest,
                                          rk_npu_w4a8_strategy_ex* fastest_strategies,
                                          rk_npu_w4a8_family_summary* stable,
                                          rk_npu_w4a8_strategy_ex* stable_strategies, int* cache_hits,
                                          int* cache_misses) {
    return family(ctx, c, B, w_scale, cache_directory, refresh, fastest, fastest_strategies, stable, stable_strategies,
                  cache_hits, cache_misses, true);
}

} // extern "C"
