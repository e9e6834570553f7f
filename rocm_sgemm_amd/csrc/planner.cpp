// Config selection: the tuned table and its lookup (the reference's generated
// detail::find_best_config / find_closest_config, config/generate_config.py:174-267), the cost
// model and the planner that choose what a call runs.  Host only: no HIP call is made here.

#include "dispatch.hpp"

#include <algorithm>
#include <climits>
#include <cmath>
#include <limits>
#include <vector>

namespace rocm_sgemm
{
namespace detail
{

#include "config_table.inc"

namespace
{

bool key_less(const tuned_entry& e, size_t m, size_t n, size_t k, int la, int lb, int lc)
{
    if(e.m != m) return e.m < m;
    if(e.n != n) return e.n < n;
    if(e.k != k) return e.k < k;
    if(e.layout_a != la) return e.layout_a < la;
    if(e.layout_b != lb) return e.layout_b < lb;
    return e.layout_c < lc;
}

// A column-major C (M x N) is computed as the row-major N x M matrix C^T = B^T * A^T with the
// operands, the problem shape and the tile shape exchanged (run_gemm), and a row-major operand is
// the transpose of a column-major one.  So the problem (M, N, K, a, b, c) under a config launches
// exactly what (N, M, K, !b, !a, !c) launches under the same config with macro_m / macro_n and
// waves_m / waves_n exchanged: an entry tuned for one is an entry for the other.
tuned_entry mirror_of(const tuned_entry& e)
{
    tuned_entry r = e;
    r.m = e.n, r.n = e.m;
    r.layout_a = 1 - e.layout_b, r.layout_b = 1 - e.layout_a, r.layout_c = 1 - e.layout_c;
    r.config.macro_m = e.config.macro_n, r.config.macro_n = e.config.macro_m;
    r.config.waves_m = e.config.waves_n, r.config.waves_n = e.config.waves_m;
    return r;
}

// The table as the library looks things up in it: every tuned entry, and the mirror image of
// every entry whose mirror was not tuned itself; sorted by key like the tuned table.
const std::vector<tuned_entry>& lookup_entries()
{
    static const std::vector<tuned_entry> entries = [] {
        std::vector<tuned_entry> v(tuned_table, tuned_table + tuned_table_size);
        const auto before = [](const tuned_entry& a, const tuned_entry& b) {
            return key_less(a, b.m, b.n, b.k, b.layout_a, b.layout_b, b.layout_c);
        };
        for(int i = 0; i < tuned_table_size; ++i)
        {
            const tuned_entry m = mirror_of(tuned_table[i]);
            // (the tuned table is sorted: binary search)
            const tuned_entry* at = std::lower_bound(tuned_table, tuned_table + tuned_table_size, m, before);
            if(at == tuned_table + tuned_table_size || before(m, *at)) v.push_back(m);
        }
        std::sort(v.begin(), v.end(), before);
        return v;
    }();
    return entries;
}

// Distance between two problem sizes: sum of squared log2 ratios (the reference's measure).  The
// logarithms of the built-in table's sizes are computed once per process, those of a problem once
// per lookup: a lookup scans the table up to three times.
struct log_size
{
    double m, n, k;
};

log_size logs_of(size_t m, size_t n, size_t k)
{
    return log_size{std::log2(static_cast<double>(m)), std::log2(static_cast<double>(n)),
                    std::log2(static_cast<double>(k))};
}

double log2_distance(const log_size& a, const log_size& b)
{
    const double dm = a.m - b.m, dn = a.n - b.n, dk = a.k - b.k;
    return dm * dm + dn * dn + dk * dk;
}

const log_size* builtin_logs()
{
    static const std::vector<log_size> logs = [] {
        std::vector<log_size> v;
        for(const tuned_entry& e : lookup_entries())
            v.push_back(logs_of(e.m, e.n, e.k));
        return v;
    }();
    return logs.data();
}

} // namespace

const rocm_sgemm_config& select_config(const tuned_entry*       table,
                                       int                      table_size,
                                       const rocm_sgemm_config& fallback,
                                       size_t                   m,
                                       size_t                   n,
                                       size_t                   k,
                                       int                      la,
                                       int                      lb,
                                       int                      lc)
{
    if(table_size <= 0)
    {
        return fallback;
    }
    // Exact hit by binary search over the key-sorted table.
    int lo = 0, hi = table_size;
    while(lo < hi)
    {
        const int mid = lo + (hi - lo) / 2;
        if(key_less(table[mid], m, n, k, la, lb, lc))
            lo = mid + 1;
        else
            hi = mid;
    }
    if(lo < table_size)
    {
        const tuned_entry& e = table[lo];
        if(e.m == m && e.n == n && e.k == k && e.layout_a == la && e.layout_b == lb
           && e.layout_c == lc)
        {
            return e.config;
        }
    }
    // Nearest size among entries tuned for the same three layouts; first minimum wins.  Problems
    // whose M, N and K are multiples of 4 have 16-byte aligned operand lines in every layout and
    // run the direct-to-LDS kernels with 16-byte loads (masked ones if a dimension is ragged); all
    // others run the masked kernels with 4-byte loads, and the best tile shapes of the two kinds
    // differ.  So entries of the problem's own kind are searched first (the
    // reference's table holds powers of two only and never meets the distinction).
    double          best     = std::numeric_limits<double>::max();
    int             best_idx = -1;
    const log_size  here     = logs_of(m, n, k);
    const log_size* known    = table == lookup_entries().data() ? builtin_logs() : nullptr; // else a caller's own table
    const auto      entry_logs = [&](int i) { return known ? known[i] : logs_of(table[i].m, table[i].n, table[i].k); };
    const auto whole = [](size_t a, size_t b, size_t c) { return a % 4 == 0 && b % 4 == 0 && c % 4 == 0; };
    for(int same_kind = 1; same_kind >= 0 && best_idx < 0; --same_kind)
    {
        for(int i = 0; i < table_size; ++i)
        {
            const tuned_entry& e = table[i];
            if(e.layout_a == la && e.layout_b == lb && e.layout_c == lc
               && (!same_kind || whole(e.m, e.n, e.k) == whole(m, n, k)))
            {
                const double d = log2_distance(here, entry_logs(i));
                if(d < best)
                {
                    best     = d;
                    best_idx = i;
                }
            }
        }
    }
    if(best_idx >= 0)
    {
        return table[best_idx].config;
    }
    // Nearest size of any layout.
    for(int i = 0; i < table_size; ++i)
    {
        const double d = log2_distance(here, entry_logs(i));
        if(d < best)
        {
            best     = d;
            best_idx = i;
        }
    }
    return best_idx >= 0 ? table[best_idx].config : fallback;
}

namespace
{

constexpr long long model_cus = 256; // the library is built and tuned for MI355X

// A split_k tuned for a neighbour of another size suits that neighbour's number of tiles.  Few
// workgroups in all -> no uniform split, the stream-K tail deals the K range of the tiles out to
// every CU; far more workgroups than CUs -> split less, the partial products are pure overhead
// once the grid is full.
void fit_split(rocm_sgemm_config& c, size_t m, size_t n, size_t k, size_t batch)
{
    if(c.split_k <= 1 || c.macro_m <= 0 || c.macro_n <= 0 || c.k_tile <= 0) return;
    const unsigned long long tiles
        = static_cast<unsigned long long>((m + c.macro_m - 1) / c.macro_m) * ((n + c.macro_n - 1) / c.macro_n) * batch;
    const unsigned long long k_tiles = (k + c.k_tile - 1) / c.k_tile;
    if(tiles * c.split_k * 4 <= model_cus * 3 && k_tiles >= 8 && batch == 1) // the tail needs one product
    {
        c.split_k    = 1;
        c.wave_slots = 0;
    }
    else if(tiles * c.split_k > 4 * model_cus)
    {
        const unsigned long long want = (2 * model_cus + tiles - 1) / tiles;
        c.split_k = static_cast<int>(want < 1 ? 1 : (want < static_cast<unsigned long long>(c.split_k) ? want : c.split_k));
    }
}

} // namespace

// Whether run_gemm deals the last wave of tiles out as a stream-K tail, and over how many slots.
// One rule, used by the launch and by the cost model below.
bool tail_applies(const rocm_sgemm_config& c, long long tiles, long long k_tiles, size_t k, long long cus,
                  long long* slots_out, long long* r_out)
{
    const int       waves  = c.waves_m * c.waves_n * (c.waves_k > 1 ? c.waves_k : 1);
    const int       per_cu = waves >= 4 ? 1 : 4 / (waves < 1 ? 1 : waves); // workgroups that fill a CU's four SIMDs
    const long long slots  = c.wave_slots > 1 ? c.wave_slots : cus * per_cu;
    const long long r      = tiles % slots;
    // one tile on its share of a CU at ~90 % of 157.3 TFLOP/s / 256 CUs, in microseconds
    const double tile_us  = 2.0 * c.macro_m * c.macro_n * static_cast<double>(k) / 553.0e3 * per_cu;
    const double saved_us = tile_us * (1.0 - static_cast<double>(r) / static_cast<double>(slots));
    if(slots_out) *slots_out = slots;
    if(r_out) *r_out = r;
    return c.split_k == 1 && c.wave_slots != 1 && k_tiles >= 8 && r > 0 && 100 * r <= 85 * slots
           && (c.wave_slots > 1 || saved_us >= 12.0) && r * k_tiles <= INT_MAX;
}

// Rough duration of a problem under a config, in microseconds.  Structure: tiles are dealt out in
// waves of one workgroup-set per CU; a tile takes the larger of its matrix-pipe time (at the
// sustained efficiency of its wave-tile size) and the time its operand panels take from L2 into
// LDS (small tiles are bound by that: a 64 x 64 tile needs 16 bytes per 256 flop); the stream-K tail
// or the K split add their second pass; every round of tiles exposes what a workgroup loads
// before its first MFMA (stages - 1 K-tiles); every launch a fixed cost.  The constants are a
// least-squares fit (log time, weighted towards each problem's fastest configs) to tuner sweeps of
// the whole family over 79 problems between 192 x 192 x 8192 and 7052 x 2436 x 856, regular and
// ragged, on MI355X (6 424 timed configs); choosing each problem's config by this model lands
// within 3.9 % of its fastest on average (3.1 - 4.5 % on held-out thirds, worst case 23 %; without
// the fill term 4.5 %, 3.7 - 6.3 % and 30 %).  Since the main loop lost its stalls the efficiencies
// of all wave-tile sizes are within 3 % of each other.  Used to choose among candidate configs
// for problems that are not table entries, so mainly the ordering matters.
double predict_us(const rocm_sgemm_config& c, size_t m, size_t n, size_t k, size_t batch)
{
    const int    waves     = c.waves_m * c.waves_n * (c.waves_k > 1 ? c.waves_k : 1);
    const int    per_cu    = waves >= 4 ? 1 : 4 / (waves < 1 ? 1 : waves);
    const double wave_area = static_cast<double>(c.macro_m / c.waves_m) * (c.macro_n / c.waves_n);
    double       eff = wave_area >= 8192 ? 0.989 : wave_area >= 4096 ? 0.984 : wave_area >= 2048 ? 1.000 : 0.971;
    if(c.k_tile >= 64) eff *= 0.982;
    if(c.mfma == 16) eff *= 0.933;
    if(c.stages == 0) eff *= 1.032;
    if(c.stages >= 3) eff *= 0.985;
    // ragged problems run the masked kernels: 16-byte loads when every dimension is a multiple
    // of 4, 4-byte loads otherwise
    const bool aligned = m % 4 == 0 && n % 4 == 0 && k % 4 == 0;
    const bool full    = m % c.macro_m == 0 && n % c.macro_n == 0 && k % c.k_tile == 0;
    if(!aligned)
        eff *= 0.861;
    else if(!full)
        eff *= 0.930;
    // the products of a batch are one launch: their tiles fill the waves together
    const long long tiles   = static_cast<long long>((m + c.macro_m - 1) / c.macro_m) * ((n + c.macro_n - 1) / c.macro_n)
                              * static_cast<long long>(batch);
    const long long k_tiles = static_cast<long long>((k + c.k_tile - 1) / c.k_tile);
    const double    kd      = static_cast<double>(k);
    const double    compute = 2.0 * c.macro_m * c.macro_n * kd / (614.5e3 * eff); // one CU's matrix pipes
    // L2 -> LDS: 40 TB/s over the CUs (the fit's upper bound: with 16-byte loads this term no longer
    // binds any shape of the family); 11.75 TB/s for the 4-byte loads of a direct-to-LDS shape,
    // which are bound by the number of load instructions
    const double    l2_tbs  = !aligned && c.stages != 0 ? 11.75 : 40.0;
    const double    panels  = (c.macro_m + c.macro_n) * kd * 4.0 / (l2_tbs * 1.0e6 / model_cus);
    const double    tile_us = std::sqrt(std::sqrt(compute * compute * compute * compute + panels * panels * panels * panels)) * per_cu;
    const double    out_mb  = static_cast<double>(m) * n * 4.0 / 1.0e6 * static_cast<double>(batch);
    // what a workgroup loads before its first MFMA (stages - 1 K-tiles of both panels), in KiB:
    // nothing overlaps it at the start of a round of tiles; 0.0281 us per KiB = 36 GB/s per CU
    const double    fill_kb = ((c.stages > 2 ? c.stages : 2) - 1) * static_cast<double>(c.k_tile)
                              * (c.macro_m + c.macro_n) * 4.0 / 1024.0;
    const double    fill_us = 0.0281 * fill_kb;
    double          t       = 4.44; // launch, last stores
    if(c.split_k > 1)
    {
        const long long split  = c.split_k < k_tiles ? c.split_k : k_tiles;
        const long long groups = tiles * split;
        const long long slots  = model_cus * per_cu;
        t += static_cast<double>((groups + slots - 1) / slots) * (tile_us / split + fill_us);
        t += 2.57 + (split + 1) * out_mb / 4.15; // second pass: launch gap, partials at ~4 TB/s
        return t;
    }
    long long slots = 0, r = 0;
    const bool tail = tail_applies(c, tiles, k_tiles, k, model_cus, &slots, &r) && batch == 1;
    t += static_cast<double>(tiles / slots) * tile_us + static_cast<double>((tiles + slots - 1) / slots) * fill_us;
    if(r > 0)
    {
        if(tail)
        {
            const double tile_mb = c.macro_m * c.macro_n * 4.0 / 1.0e6;
            // second pass: launch gap, the segments at ~5 TB/s
            t += tile_us * static_cast<double>(r) / slots + 6.15 + (2.0 * slots + r) * tile_mb / 5.10;
        }
        else
        {
            t += tile_us;
        }
    }
    return t;
}

namespace
{
rocm_sgemm_config plan_uncached(size_t m, size_t n, size_t k, int la, int lb, int lc, size_t batch);
}

// Planning costs a few microseconds for a problem that is not a table entry; callers usually
// work through a handful of shapes again and again (the layers of a model, the steps of a
// factorisation), so every thread remembers its last sixteen answers (the tables never change).
// Sixteen slots, replaced in turn: a lookup is a scan of at most sixteen keys.
rocm_sgemm_config plan_config(size_t m, size_t n, size_t k, int la, int lb, int lc, size_t batch)
{
    struct memo
    {
        size_t            m = 0, n = 0, k = 0, batch = 0;
        int               la = -1, lb = -1, lc = -1;
        rocm_sgemm_config config{};
    };
    constexpr int          slots = 16;
    thread_local memo      remembered[slots];
    thread_local int       used = 0, next = 0;
    for(int i = 0; i < used; ++i)
    {
        const memo& e = remembered[i];
        if(e.m == m && e.n == n && e.k == k && e.batch == batch && e.la == la && e.lb == lb && e.lc == lc)
        {
            return e.config;
        }
    }
    memo& e  = remembered[next];
    e.config = plan_uncached(m, n, k, la, lb, lc, batch < 1 ? 1 : batch);
    e.m = m, e.n = n, e.k = k, e.batch = batch, e.la = la, e.lb = lb, e.lc = lc;
    next = next + 1 == slots ? 0 : next + 1;
    used = used < slots ? used + 1 : slots;
    return e.config;
}

namespace
{

rocm_sgemm_config plan_uncached(size_t m, size_t n, size_t k, int la, int lb, int lc, size_t batch)
{
    const tuned_entry* table      = lookup_table();
    const int          table_size = lookup_table_size();
    const rocm_sgemm_config nearest = select_config(table, table_size, default_config, m, n, k, la, lb, lc);
    // (the table is tuned on single products: a batch of them is planned like any other problem)
    for(int i = 0; i < table_size && batch == 1; ++i)
    {
        const tuned_entry& e = table[i];
        if(e.m == m && e.n == n && e.k == k && e.layout_a == la && e.layout_b == lb && e.layout_c == lc)
        {
            return nearest; // tuned for exactly this problem (or for its mirror image)
        }
    }
    // Not a table entry.  The nearest entry's config (split_k fitted to this problem) is the
    // reference's answer, but the log-distance rule is blind to how a tile shape divides this
    // problem's M and N and to how many tiles that leaves for 256 CUs.  So the cost model also
    // prices the configs of the four nearest entries of the same layouts and kind, and every
    // direct-to-LDS tile shape of the family with 32 x 32 MFMAs and tiles of at least 64 x 64 (or
    // smaller ones with waves along K, which keep a large wave tile; the 16-row tiles of 16 x 16
    // MFMAs where the problem has at most 16 rows or columns) at
    // split_k 1, 2, 3, 4, 6 and 8; the cheapest of them replaces the nearest entry's config only if
    // the model expects it to be at least 5 % faster (above the model's error of 3 - 4.5 % on held-out problems).
    const auto aligned_kind = [](size_t a, size_t b, size_t c) { return a % 4 == 0 && b % 4 == 0 && c % 4 == 0; };
    constexpr int   max_candidates = 4;
    const log_size  here  = logs_of(m, n, k);
    const log_size* known = builtin_logs();
    int           idx[max_candidates];
    double        dist[max_candidates];
    int           count = 0;
    for(int i = 0; i < table_size; ++i)
    {
        const tuned_entry& e = table[i];
        if(e.layout_a != la || e.layout_b != lb || e.layout_c != lc
           || aligned_kind(e.m, e.n, e.k) != aligned_kind(m, n, k))
        {
            continue;
        }
        const double d = log2_distance(here, known[i]);
        int          pos = count < max_candidates ? count : max_candidates;
        while(pos > 0 && d < dist[pos - 1]) --pos; // strict: the first of equals stays first
        if(pos >= max_candidates) continue;
        const int last = count < max_candidates ? count : max_candidates - 1;
        for(int j = last; j > pos; --j)
        {
            idx[j]  = idx[j - 1];
            dist[j] = dist[j - 1];
        }
        idx[pos]  = i;
        dist[pos] = d;
        if(count < max_candidates) ++count;
    }
    rocm_sgemm_config best = nearest;
    fit_split(best, m, n, k, batch);
    double       best_us    = predict_us(best, m, n, k, batch);
    const double nearest_us = best_us;
    const auto   consider   = [&](const rocm_sgemm_config& c) {
        const double us = predict_us(c, m, n, k, batch);
        if(us < best_us && us <= 0.95 * nearest_us)
        {
            best    = c;
            best_us = us;
        }
    };
    for(int j = 0; j < count; ++j)
    {
        rocm_sgemm_config c = table[idx[j]].config;
        fit_split(c, m, n, k, batch);
        consider(c);
    }
    for(int i = 0; i < family_size(); ++i)
    {
        rocm_sgemm_config s{};
        family_entry(i, &s);
        if(s.stages < 2 || ((s.macro_m < 64 || s.macro_n < 64) && s.waves_k <= 1)) continue;
        // 16-row (16-column) tiles of 16 x 16 MFMAs: only where the problem has no more rows (columns)
        if(s.mfma != 32 && !((s.macro_m == 16 && m <= 16) || (s.macro_n == 16 && n <= 16))) continue;
        const long long k_tiles = static_cast<long long>((k + s.k_tile - 1) / s.k_tile);
        for(const int split : {1, 2, 3, 4, 6, 8})
        {
            if(split > 1 && k_tiles < 2LL * split) break; // at least two K-tiles per slice
            consider(rocm_sgemm_config{s.macro_m, s.macro_n, s.k_tile, s.waves_m, s.waves_n, s.mfma, s.stages,
                                       split, 4, 0, s.waves_k});
        }
    }
    return best;
}

} // namespace

const tuned_entry* builtin_table()
{
    return tuned_table;
}

const tuned_entry* lookup_table()
{
    return lookup_entries().data();
}

int lookup_table_size()
{
    return static_cast<int>(lookup_entries().size());
}

int builtin_table_size()
{
    return tuned_table_size;
}

const rocm_sgemm_config& builtin_default()
{
    return default_config;
}
} // namespace detail
} // namespace rocm_sgemm
