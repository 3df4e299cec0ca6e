// Tactic profiler: times the candidate kernels / launch shapes of a problem on the device and
// keeps the fastest per row count.  Counterpart of GemmPluginProfiler::profileTactics
// (plugins/common/gemmPluginProfiler.cpp:118-216: every m in [minM, 15], then powers of two;
// timing loop :329-367; lookup by exact m, then the next profiled m, :221-250) and of the tactic map
// the reference plugins serialise into an engine (weightOnlyQuantMatmulPlugin.cpp:374-391).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <map>
#include <mutex>
#include <shared_mutex>
#include <string>
#include <tuple>
#include <vector>

#include "woq_internal.h"

namespace woq
{
namespace
{
thread_local Tactic const* tl_tactic = nullptr;

// n, k, quant_algo, group_size, out_dtype, m
using Key = std::tuple<int, int, int, int, int, int>;

std::shared_timed_mutex g_mutex;
std::map<Key, Tactic> g_table;
std::atomic<int> g_entries{0};

Key key_of(woq_matmul_args const& a, int m)
{
    return Key{a.n, a.k, a.quant_algo, a.group_size, a.out_dtype, m};
}

bool same_problem(Key const& a, Key const& b)
{
    return std::get<0>(a) == std::get<0>(b) && std::get<1>(a) == std::get<1>(b) && std::get<2>(a) == std::get<2>(b)
        && std::get<3>(a) == std::get<3>(b) && std::get<4>(a) == std::get<4>(b);
}

bool valid_tactic(Tactic const& t)
{
    if (t.regime == WOQ_REGIME_AUTO) // "as the heuristics choose": profiled, and nothing was clearly faster
        return true;
    if (t.regime == WOQ_REGIME_STREAM)
        return t.ns >= 1 && t.waves >= 1 && t.pf >= 1 && t.lds >= 0 && t.lds <= 2
            && (t.mt == 1 || t.mt == 2 || t.mt == 4 || t.mt == 8);
    if (t.regime == WOQ_REGIME_GEMM)
        return t.k_splits >= 1 && (t.skinny ? (t.rt == 2 || t.rt == 4) : (t.rt == 4 || t.rt == 8 || t.rt == 16));
    return false;
}

void store(Key const& key, Tactic const& t)
{
    std::unique_lock<std::shared_timed_mutex> lock(g_mutex);
    g_table[key] = t;
    g_entries.store((int) g_table.size());
}

int describe(Tactic const& t, char* buf, size_t len)
{
    if (t.regime == WOQ_REGIME_AUTO)
        return std::snprintf(buf, len, "heuristic");
    if (t.regime == WOQ_REGIME_STREAM)
        return std::snprintf(buf, len, "stream mt=%d ns=%d waves=%d pf=%d lds=%d", t.mt, t.ns, t.waves, t.pf, t.lds);
    return std::snprintf(buf, len, "gemm %s rt=%d splits=%d", t.skinny ? "skinny" : "exact", t.rt, t.k_splits);
}

// 16-row tiles per wavefront the streaming kernel is instantiated with for m rows
int stream_mt(int m)
{
    return m <= 16 ? 1 : (m <= 32 ? 2 : (m <= 64 ? 4 : 8));
}

std::vector<Tactic> candidates(woq_matmul_args const& a, bool stream_allowed)
{
    std::vector<Tactic> c;
    int const bits = (a.quant_algo & WOQ_ALGO_INT8_WEIGHT) ? 8 : 4;
    int const m = a.m;
    if (stream_allowed && m <= kStreamMaxM)
    {
        int const mt = stream_mt(m);
        int const l = a.group_size != 0 ? 2 : 0;
        auto add = [&](int ns, int waves, int pf, int lds) {
            c.push_back(Tactic{WOQ_REGIME_STREAM, mt, ns, waves, pf, lds, 0, 0, 0});
        };
        if (mt == 1)
        {
            add(1, 8, 4, 1), add(2, 8, 4, 1), add(3, 8, 2, 1), add(4, 8, 2, 1); // a shape whose operands do not fit the LDS is skipped
            add(1, 8, 4, l), add(2, 8, 2, l), add(4, 4, 2, l);
        }
        else if (mt == 2)
            add(2, 8, 2, 0), add(1, 8, 2, 0), add(2, 8, 2, l), add(1, 8, 2, l);
        else if (mt == 4)
            add(1, 8, 1, 0), add(2, 8, 1, 0), add(1, 8, 1, l), add(2, 8, 1, l);
        else
            add(1, 4, 1, 0), add(1, 8, 1, 0);
    }
    if (m > 8)
    {
        int const tk = tile_k_of_bits(bits);
        int const k_tiles = (a.k + tk - 1) / tk;
        auto add = [&](bool skinny, int rt) {
            long const tiles = gemm_tiles(m, a.n, rt);
            int s = 1;
            (void) gemm_best_split(skinny, rt, tiles, m, a.n, a.k, bits, true, s);
            int const cap = k_tiles / 4 > 1 ? k_tiles / 4 : 1;
            // around the cost model's split, and the largest that still runs as one round of workgroups
            std::vector<int> splits{1, s - 1, s, s + 1, s * 3 / 4, (int) (256 / tiles), (int) (224 / tiles)};
            std::sort(splits.begin(), splits.end());
            splits.erase(std::unique(splits.begin(), splits.end()), splits.end());
            for (int v : splits)
                if (v >= 1 && v <= cap)
                    c.push_back(Tactic{WOQ_REGIME_GEMM, 0, 0, 0, 0, 0, skinny ? 1 : 0, rt, v});
        };
        if (bits == 4 && m <= 32)
            add(true, 2);
        add(true, 4);
        add(false, 4);
        if (m > 64)
            add(false, 8);
        if (m > 128)
            add(false, 16);
    }
    return c;
}

} // namespace

Tactic const* current_tactic()
{
    return tl_tactic;
}

TacticScope::TacticScope(Tactic const* t)
    : prev(tl_tactic)
{
    tl_tactic = t;
}

TacticScope::~TacticScope()
{
    tl_tactic = prev;
}

bool find_tactic(woq_matmul_args const& a, Tactic& out)
{
    if (g_entries.load(std::memory_order_relaxed) == 0)
        return false;
    std::shared_lock<std::shared_timed_mutex> lock(g_mutex);
    Key const key = key_of(a, a.m);
    auto it = g_table.lower_bound(key); // the entry of m rows, else of the next profiled row count
    if (it == g_table.end() || !same_problem(it->first, key))
        return false;
    out = it->second;
    return true;
}

size_t tuned_split_bytes(int m, int n, int k, int quant_algo)
{
    if (g_entries.load(std::memory_order_relaxed) == 0)
        return 0;
    std::shared_lock<std::shared_timed_mutex> lock(g_mutex);
    // an entry serves every row count from the previous profiled one up to its own
    size_t bytes = 0;
    for (auto const& e : g_table)
    {
        Key const& key = e.first;
        if (std::get<0>(key) == n && std::get<1>(key) == k && std::get<2>(key) == quant_algo
            && e.second.regime == WOQ_REGIME_GEMM && e.second.k_splits > 1)
        {
            int const rows = std::get<5>(key) < m ? std::get<5>(key) : m;
            size_t const b = split_partial_bytes(rows, n, e.second.k_splits);
            bytes = b > bytes ? b : bytes;
        }
    }
    return bytes;
}

} // namespace woq

using namespace woq;

extern "C" int woq_profile_tactics(const woq_matmul_args* args, int32_t min_m, int32_t max_m, void* stream)
{
    if (!args)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "args is NULL");
    if (min_m < 1 || max_m < min_m)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "profile range [%d, %d] is empty", min_m, max_m);
    if (args->quant_algo & WOQ_ALGO_FP8_ALPHA)
        return WOQ_OK; // W4A8 has one kernel per regime: nothing to choose between
    woq_matmul_args a = *args;
    a.regime = WOQ_REGIME_AUTO;
    a.m = max_m;
    {
        TacticScope none(nullptr);
        if (int rc = woq_matmul_check(&a)) // the buffers are taken to hold max_m rows
            return rc;
    }
    hipStream_t const s = static_cast<hipStream_t>(stream);
    // weights of real models are never in the last-level cache when a layer runs: evict between runs
    size_t const flush_bytes = (size_t) 512 << 20;
    void* flush = nullptr;
    hipEvent_t t0 = nullptr, t1 = nullptr;
    if (hipMalloc(&flush, flush_bytes) != hipSuccess || hipEventCreate(&t0) != hipSuccess
        || hipEventCreate(&t1) != hipSuccess)
    {
        (void) hipGetLastError();
        if (flush)
            (void) hipFree(flush);
        if (t0)
            (void) hipEventDestroy(t0);
        return fail(WOQ_ERR_RUNTIME, "profiling needs a 512 MiB scratch allocation and two events");
    }
    std::vector<int> rows;
    for (int m = min_m; m <= max_m && m <= 15; ++m)
        rows.push_back(m);
    for (int m = 16; m < max_m; m *= 2)
        if (m >= min_m)
            rows.push_back(m);
    if (max_m > 15)
        rows.push_back(max_m);

    // Time of one candidate: the three fastest of five runs after a warm-up, each after an eviction
    // of the last-level cache.  Negative: the candidate does not run on this problem.
    constexpr int kWarmup = 1, kRuns = 5, kKept = 3;
    auto time_tactic = [&](Tactic const& t) -> float {
        TacticScope scope(&t);
        if (woq_matmul_check(&a) != WOQ_OK)
            return -1.f; // e.g. the workspace given does not cover this split
        float ms[kRuns];
        for (int r = 0; r < kWarmup + kRuns; ++r)
        {
            float v = 0.f;
            bool const ok = hipMemsetAsync(flush, r, flush_bytes, s) == hipSuccess && hipEventRecord(t0, s) == hipSuccess
                && woq_matmul(&a, stream) == WOQ_OK && hipEventRecord(t1, s) == hipSuccess
                && hipEventSynchronize(t1) == hipSuccess && hipEventElapsedTime(&v, t0, t1) == hipSuccess;
            if (!ok)
            {
                (void) hipGetLastError();
                return -1.f;
            }
            if (r >= kWarmup)
                ms[r - kWarmup] = v;
        }
        std::sort(ms, ms + kRuns);
        float total = 0.f;
        for (int r = 0; r < kKept; ++r)
            total += ms[r];
        return total;
    };
    // A candidate replaces the heuristics' own choice only when it is clearly faster: differences
    // of a few percent are within what the same launch varies by from run to run.
    constexpr float kClearlyFaster = 0.96f;
    Tactic const heuristic{WOQ_REGIME_AUTO, 0, 0, 0, 0, 0, 0, 0, 0};
    bool gemm_won = false;
    int rc_out = WOQ_OK;
    for (int m : rows)
    {
        a.m = m;
        float const heuristic_ms = time_tactic(heuristic);
        Tactic best = heuristic;
        float best_ms = heuristic_ms;
        for (Tactic const& t : candidates(a, !(gemm_won && m > 16)))
        {
            float const ms = time_tactic(t);
            if (ms < 0.f)
                continue;
            if (best_ms < 0.f || (ms < best_ms && (heuristic_ms < 0.f || ms < kClearlyFaster * heuristic_ms)))
            {
                best_ms = ms;
                best = t;
            }
        }
        if (best_ms < 0.f)
        {
            rc_out = fail(WOQ_ERR_RUNTIME, "no tactic ran for m = %d", m);
            break;
        }
        if (m >= 16 && (best.regime == WOQ_REGIME_GEMM
                || (best.regime == WOQ_REGIME_AUTO && woq_select_regime(m, a.n, a.k, a.quant_algo) == WOQ_REGIME_GEMM)))
            gemm_won = true;
        store(key_of(a, m), best);
    }
    (void) hipStreamSynchronize(s);
    (void) hipFree(flush);
    (void) hipEventDestroy(t0);
    (void) hipEventDestroy(t1);
    return rc_out;
}

extern "C" int woq_tactic_count(void)
{
    return g_entries.load();
}

extern "C" void woq_clear_tactics(void)
{
    std::unique_lock<std::shared_timed_mutex> lock(g_mutex);
    g_table.clear();
    g_entries.store(0);
}

extern "C" int woq_describe_tactic(const woq_matmul_args* args, char* buf, size_t len)
{
    if (!args || !buf || len == 0)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "args and a buffer are required");
    Tactic t;
    if (args->regime == WOQ_REGIME_AUTO && find_tactic(*args, t))
        describe(t, buf, len);
    else
        std::snprintf(buf, len, "heuristic");
    return WOQ_OK;
}

extern "C" size_t woq_export_tactics(char* buf, size_t len)
{
    std::string text = "woq-tactics 1\n";
    {
        std::shared_lock<std::shared_timed_mutex> lock(g_mutex);
        for (auto const& e : g_table)
        {
            Key const& k = e.first;
            Tactic const& t = e.second;
            char line[160];
            std::snprintf(line, sizeof line, "%d %d %d %d %d %d %d %d %d %d %d %d %d %d %d\n", std::get<0>(k),
                std::get<1>(k), std::get<2>(k), std::get<3>(k), std::get<4>(k), std::get<5>(k), t.regime, t.mt, t.ns,
                t.waves, t.pf, t.lds, t.skinny, t.rt, t.k_splits);
            text += line;
        }
    }
    if (buf && len > text.size())
        std::memcpy(buf, text.c_str(), text.size() + 1);
    return text.size() + 1;
}

extern "C" int woq_import_tactics(const char* text)
{
    if (!text)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "text is NULL");
    int version = 0, used = 0;
    if (std::sscanf(text, "woq-tactics %d\n%n", &version, &used) != 1 || version != 1)
        return fail(WOQ_ERR_INVALID_ARGUMENT, "not a tactic table of this library (header 'woq-tactics 1' expected)");
    std::vector<std::pair<Key, Tactic>> parsed;
    char const* at = text + used;
    while (*at)
    {
        int v[15], n = 0;
        if (std::sscanf(at, "%d %d %d %d %d %d %d %d %d %d %d %d %d %d %d\n%n", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5],
                &v[6], &v[7], &v[8], &v[9], &v[10], &v[11], &v[12], &v[13], &v[14], &n)
                != 15
            || n == 0)
            return fail(WOQ_ERR_INVALID_ARGUMENT, "malformed tactic line %zu", parsed.size() + 1);
        Tactic const t{v[6], v[7], v[8], v[9], v[10], v[11], v[12], v[13], v[14]};
        if (v[0] <= 0 || v[1] <= 0 || v[5] <= 0 || !valid_tactic(t))
            return fail(WOQ_ERR_INVALID_ARGUMENT, "tactic line %zu names no kernel of this library", parsed.size() + 1);
        parsed.push_back({Key{v[0], v[1], v[2], v[3], v[4], v[5]}, t});
        at += n;
    }
    for (auto const& e : parsed) // all or nothing
        store(e.first, e.second);
    return WOQ_OK;
}
