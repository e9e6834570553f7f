// Trial binary of the tuner: times one config (or sweeps the whole precompiled family) for one
// problem and prints the result.  Same role as the reference's `tuner`
// (reference rocm_sgemm/config/tuner.cpp:440-512: positional M N K, config ints, layout ints), but
// a trial is a plain library call - rocm_sgemm_f32_with_config - because every tile shape of the
// search space is compiled into librocm_sgemm; nothing is compiled at run time.
//
//   tuner M N K macro_m macro_n k_tile waves_m waves_n mfma stages split_k group_m wave_slots waves_k partial_sums A B C [iters] [warmup]
//       layouts: 0 = row_major, 1 = col_major.  Prints "time: <avg> ms  min: <min> ms ...".
//   tuner --sweep M N K A B C [--iters n] [--warmup n] [--splits a,b,..] [--groups a,b,..] [--slots a,b,..] [--sums a,b]
//       one line per (tile shape, split_k, group_m, ..):  "cfg <12 ints> avg_ms <..> min_ms <..> tflops <..> ok <0|1>"
//
// Inputs are uniform[-1, 1) from a fixed xorshift stream; every trial is checked on 256 sampled
// entries against an fp64 dot product so that a mis-tuned config can never enter the table.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include <hip/hip_runtime.h>
#include <rocm_sgemm.h>

#include "../benchmark/sampled_check.hpp"

#define CHECK_HIP(call)                                                                      \
    do                                                                                       \
    {                                                                                        \
        hipError_t status_ = (call);                                                         \
        if(status_ != hipSuccess)                                                            \
        {                                                                                    \
            std::fprintf(stderr, "HIP error %d (%s) at %s:%d\n", static_cast<int>(status_),  \
                         hipGetErrorString(status_), __FILE__, __LINE__);                    \
            std::exit(EXIT_FAILURE);                                                         \
        }                                                                                    \
    } while(0)

namespace
{

struct problem
{
    size_t             M, N, K;
    int                la, lb, lc;
    std::vector<float> hA, hB;
    float *            dA = nullptr, *dB = nullptr, *dC = nullptr;
    hipStream_t        stream = nullptr;
};

uint64_t rng_state = 0x9E3779B97F4A7C15ull;
float    next_uniform()
{
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return static_cast<float>(static_cast<int32_t>(rng_state >> 40) - (1 << 23)) / static_cast<float>(1 << 23);
}

void setup(problem& p)
{
    p.hA.resize(p.M * p.K);
    p.hB.resize(p.K * p.N);
    for(auto& v : p.hA) v = next_uniform();
    for(auto& v : p.hB) v = next_uniform();
    CHECK_HIP(hipStreamCreate(&p.stream));
    CHECK_HIP(hipMalloc(&p.dA, p.hA.size() * sizeof(float)));
    CHECK_HIP(hipMalloc(&p.dB, p.hB.size() * sizeof(float)));
    CHECK_HIP(hipMalloc(&p.dC, p.M * p.N * sizeof(float)));
    CHECK_HIP(hipMemcpy(p.dA, p.hA.data(), p.hA.size() * sizeof(float), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(p.dB, p.hB.data(), p.hB.size() * sizeof(float), hipMemcpyHostToDevice));
}

void teardown(problem& p)
{
    CHECK_HIP(hipFree(p.dA));
    CHECK_HIP(hipFree(p.dB));
    CHECK_HIP(hipFree(p.dC));
    CHECK_HIP(hipStreamDestroy(p.stream));
}

// Sampled check: 256 entries (corners included) against an fp64 dot product; inputs are in
// [-1, 1), so the error is scaled by K alone.  A NaN sample (C is pre-filled with NaN, so also an
// output that was never written) fails the check.
bool verify(const problem& p)
{
    std::vector<float> hC(p.M * p.N);
    CHECK_HIP(hipMemcpy(hC.data(), p.dC, hC.size() * sizeof(float), hipMemcpyDeviceToHost));
    const double worst = rocm_sgemm::check::worst_sampled_abs_error(
        hC.data(), p.hA.data(), p.hB.data(), p.M, p.N, p.K, p.la == ROCM_SGEMM_COL_MAJOR,
        p.lb == ROCM_SGEMM_COL_MAJOR, p.lc == ROCM_SGEMM_COL_MAJOR);
    return rocm_sgemm::check::within_tolerance(worst / static_cast<double>(p.K));
}

constexpr double warmup_min_ms = 40.0;
constexpr double warmup_max_ms = 600.0;

struct timing
{
    double avg_ms, min_ms;
    bool   launched, correct;
};

timing run_trial(problem& p, const rocm_sgemm_config& cfg, int iters, int warmup)
{
    timing     r{0.0, 1e30, false, false};
    hipEvent_t e0, e1;
    CHECK_HIP(hipEventCreate(&e0));
    CHECK_HIP(hipEventCreate(&e1));
    CHECK_HIP(hipMemsetAsync(p.dC, 0xFF, p.M * p.N * sizeof(float), p.stream));
    const auto launch = [&]() {
        return rocm_sgemm_f32_with_config(&cfg, p.lc, p.la, p.lb, p.dC, p.dA, p.dB, p.M, p.N, p.K,
                                          p.stream);
    };
    // Warm-up is by count AND by time: after an idle gap (the start of the process, the check of
    // the previous trial) the GPU takes tens of milliseconds of sustained work to reach its full
    // clock, some kernels several hundred, and a trial timed before that is pessimistic by an
    // amount that differs from config to config (1024 x 1024 x 16384: up to 10 %, enough to rank
    // two configs the wrong way round).  So launches are queued back to back in batches of about
    // 10 ms until at least warmup_min_ms have passed and two batches in a row agree within 1 %
    // (or warmup_max_ms have passed).
    if(launch() != ROCM_SGEMM_STATUS_OK)
    {
        std::fprintf(stderr, "trial rejected: %s\n", rocm_sgemm_last_error());
        CHECK_HIP(hipEventDestroy(e0));
        CHECK_HIP(hipEventDestroy(e1));
        return r;
    }
    for(int i = 1; i < warmup; ++i)
    {
        launch();
    }
    CHECK_HIP(hipStreamSynchronize(p.stream));
    double warmed_ms = 0.0, previous = -1.0;
    for(int batch = 4;;)
    {
        CHECK_HIP(hipEventRecord(e0, p.stream));
        for(int i = 0; i < batch; ++i)
        {
            launch();
        }
        CHECK_HIP(hipEventRecord(e1, p.stream));
        CHECK_HIP(hipEventSynchronize(e1));
        float ms = 0.0f;
        CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        warmed_ms += ms;
        const double per_launch = (ms > 1e-3f ? ms : 1e-3f) / batch;
        const bool   settled    = previous > 0.0 && std::fabs(per_launch - previous) <= 0.01 * previous;
        previous                = per_launch;
        if(warmed_ms >= warmup_min_ms && (settled || warmed_ms >= warmup_max_ms))
        {
            break;
        }
        const double next = 10.0 / per_launch;
        batch             = next < 2.0 ? 2 : (next > 4096.0 ? 4096 : static_cast<int>(next));
    }
    // Timed region: `iters` launches queued back to back, closed by one synchronisation - the
    // sustained rate a caller issuing GEMM after GEMM sees.  (With a host wait after every launch
    // the GPU idles between kernels, boosts its clock and favours other configs.)  The minimum is
    // taken over a few single launches timed the same way afterwards.
    // (at least 5 ms of them: thirty launches of a 20 us kernel are over before the timer's noise is)
    iters = std::max(iters, std::min(4096, static_cast<int>(5.0 / previous)));
    CHECK_HIP(hipEventRecord(e0, p.stream));
    for(int i = 0; i < iters; ++i)
    {
        launch();
    }
    CHECK_HIP(hipEventRecord(e1, p.stream));
    CHECK_HIP(hipEventSynchronize(e1));
    {
        float ms = 0.0f;
        CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        r.avg_ms = ms;
    }
    for(int i = 0; i < 3; ++i)
    {
        CHECK_HIP(hipEventRecord(e0, p.stream));
        launch();
        CHECK_HIP(hipEventRecord(e1, p.stream));
        CHECK_HIP(hipEventSynchronize(e1));
        float ms = 0.0f;
        CHECK_HIP(hipEventElapsedTime(&ms, e0, e1));
        r.min_ms = std::min<double>(r.min_ms, ms);
    }
    r.avg_ms /= iters;
    r.launched = true;
    r.correct  = verify(p);
    CHECK_HIP(hipEventDestroy(e0));
    CHECK_HIP(hipEventDestroy(e1));
    return r;
}

std::vector<int> parse_list(const char* s)
{
    std::vector<int> out;
    std::string      str(s), tok;
    size_t           pos = 0;
    while(pos <= str.size())
    {
        const size_t next = str.find(',', pos);
        tok               = str.substr(pos, next == std::string::npos ? std::string::npos : next - pos);
        if(!tok.empty()) out.push_back(std::atoi(tok.c_str()));
        if(next == std::string::npos) break;
        pos = next + 1;
    }
    return out;
}

int usage()
{
    std::fprintf(stderr,
                 "usage: tuner M N K macro_m macro_n k_tile waves_m waves_n mfma stages split_k group_m "
                 "wave_slots waves_k partial_sums A B C [iters] [warmup]\n"
                 "       tuner --sweep M N K A B C [--iters n] [--warmup n] [--splits a,b] "
                 "[--groups a,b] [--slots a,b] [--sums a,b]\n");
    return 2;
}

} // namespace

int main(int argc, char** argv)
{
    if(argc >= 8 && std::strcmp(argv[1], "--sweep") == 0)
    {
        problem p{};
        p.M = std::strtoull(argv[2], nullptr, 10);
        p.N = std::strtoull(argv[3], nullptr, 10);
        p.K = std::strtoull(argv[4], nullptr, 10);
        p.la = std::atoi(argv[5]), p.lb = std::atoi(argv[6]), p.lc = std::atoi(argv[7]);
        int              iters = 10, warmup = 2;
        std::vector<int> splits{1}, groups{4}, slots{0}, sums{0};
        for(int i = 8; i + 1 < argc; i += 2)
        {
            if(!std::strcmp(argv[i], "--iters")) iters = std::atoi(argv[i + 1]);
            else if(!std::strcmp(argv[i], "--warmup")) warmup = std::atoi(argv[i + 1]);
            else if(!std::strcmp(argv[i], "--splits")) splits = parse_list(argv[i + 1]);
            else if(!std::strcmp(argv[i], "--groups")) groups = parse_list(argv[i + 1]);
            else if(!std::strcmp(argv[i], "--slots")) slots = parse_list(argv[i + 1]);
            else if(!std::strcmp(argv[i], "--sums")) sums = parse_list(argv[i + 1]);
            else return usage();
        }
        setup(p);
        const double flops = 2.0 * p.M * p.N * p.K;
        for(int f = 0; f < rocm_sgemm_family_size(); ++f)
        {
            rocm_sgemm_config cfg;
            rocm_sgemm_family_entry(f, &cfg);
            for(int s : splits)
            {
                // splitting only pays while the grid is short of a few workgroups per CU
                const size_t tiles = ((p.M + cfg.macro_m - 1) / cfg.macro_m)
                                     * ((p.N + cfg.macro_n - 1) / cfg.macro_n);
                if(s > 1 && (static_cast<size_t>(s) * cfg.k_tile * 2 > p.K || tiles * s > 2048)) continue;
                for(int g : groups)
                for(int w : slots)
                for(int u : sums)
                {
                    if(w != 0 && s > 1) continue; // the tail split only applies without split_k
                    if(u != sums.front() && s == 1 && w == 1) continue; // no partial tiles to add up
                    cfg.split_k      = s;
                    cfg.group_m      = g;
                    cfg.wave_slots   = w;
                    cfg.partial_sums = u;
                    if(!rocm_sgemm_config_supported(&cfg, p.lc, p.la, p.lb)) continue;
                    const timing t = run_trial(p, cfg, iters, warmup);
                    if(!t.launched) continue;
                    std::printf("cfg %d %d %d %d %d %d %d %d %d %d %d %d avg_ms %.4f min_ms %.4f tflops %.2f ok %d\n",
                                cfg.macro_m, cfg.macro_n, cfg.k_tile, cfg.waves_m, cfg.waves_n,
                                cfg.mfma, cfg.stages, cfg.split_k, cfg.group_m, cfg.wave_slots, cfg.waves_k,
                                cfg.partial_sums, t.avg_ms,
                                t.min_ms,
                                flops / (t.avg_ms * 1e-3) * 1e-12, t.correct ? 1 : 0);
                    std::fflush(stdout);
                }
            }
        }
        teardown(p);
        return 0;
    }

    if(argc < 19)
    {
        return usage();
    }
    problem p{};
    p.M = std::strtoull(argv[1], nullptr, 10);
    p.N = std::strtoull(argv[2], nullptr, 10);
    p.K = std::strtoull(argv[3], nullptr, 10);
    rocm_sgemm_config cfg{std::atoi(argv[4]), std::atoi(argv[5]), std::atoi(argv[6]),
                          std::atoi(argv[7]), std::atoi(argv[8]), std::atoi(argv[9]),
                          std::atoi(argv[10]), std::atoi(argv[11]), std::atoi(argv[12]),
                          std::atoi(argv[13]), std::atoi(argv[14]), std::atoi(argv[15])};
    p.la = std::atoi(argv[16]), p.lb = std::atoi(argv[17]), p.lc = std::atoi(argv[18]);
    const int iters  = argc > 19 ? std::atoi(argv[19]) : 20;
    const int warmup = argc > 20 ? std::atoi(argv[20]) : 3;
    if(!rocm_sgemm_config_supported(&cfg, p.lc, p.la, p.lb))
    {
        std::fprintf(stderr, "unsupported config: %s\n", rocm_sgemm_last_error());
        return 3;
    }
    setup(p);
    const timing t = run_trial(p, cfg, iters, warmup);
    teardown(p);
    if(!t.launched)
    {
        return 4;
    }
    const double flops = 2.0 * p.M * p.N * p.K;
    std::printf("time: %.4f ms  min: %.4f ms  avg_tflops: %.2f  max_tflops: %.2f\n", t.avg_ms,
                t.min_ms, flops / (t.avg_ms * 1e-3) * 1e-12, flops / (t.min_ms * 1e-3) * 1e-12);
    if(!t.correct)
    {
        std::fprintf(stderr, "config produced a wrong result\n");
        return 5;
    }
    return 0;
}
