// bench_float - SGEMM benchmark of the MI355X library through the reference's public C++ entry
// point, rocm_sgemm::gemm<layout_C, layout_A, layout_B>(C, A, B, M, N, K, stream).
//
// Counterpart of the reference's benchmark/gemm/bench.cpp (run_benchmark :31-114, shape parser
// :125-173, main :189-317) with the same command line, the same eight layout combinations per
// shape in the same order, the same cyclic input pattern (benchmark/bench.hpp:15-29) and the same
// console row format, so a report script that parses the reference's output parses this one:
//
//   {A:m_layout::row_major,B:...,C:...,m:4096,n:4096,k:4096}/manual_time  <time> ms  <cpu> ms  <iters>
//       <avg_tflops>  <bytes_per_second>Gi/s  <max_time_ms>  <min_time_ms>  [pct_peak] [extensions]
//
// avg_tflops is the mean of the per-iteration TFLOP/s (reference bench.cpp:96-102), and the
// columns after the four the reference prints sort after them.  It does not need Google Benchmark:
// the iteration protocol is explicit instead (default 10 warm-up + 100 timed launches, each timed
// with an event pair on the launch stream).
//
// Extensions:
//   --identity_b        B = identity (square shapes): the timing methodology the reference's
//                       README describes; the output is checked bit-for-bit against A
//   --uniform [seed]    A, B uniform[-1, 1) from mt19937(seed) instead of the cyclic pattern
//   --warmup n --iters n
//   --layouts rrr,rcr,...   subset of layout combinations, letters in the order A, B, C
//   --verify            sampled fp64 check of every result (256 entries, scaled error <= 1e-6)
//   --cpu [threads]     times the reference's CPU loop nest (test/test.hpp:30-45: i-j-k, fp32
//                       accumulator) on the host at the first shape (capped at 1024^3) and prints
//                       it as a baseline row
//   --vendor            adds a rocBLAS and a hipBLASLt row per layout for context (the reference's
//                       rocblas_wrapper/src/gemm.cpp:45-58 serves column-major C only; here
//                       row-major C is served too, as the column-major C^T = B^T A^T)
//   --counters          after the timing table, hardware counters per row: the program starts
//                       `rocprofv3 --pmc <set> -- bench_float --pmc ...` (itself, one row, one
//                       counter set at a time; this process does not touch the GPU in that phase)
//                       and prints matrix-pipe busy %, LDS bank-conflict % and achieved HBM GB/s
//   --host_cost         what a call costs on the host (no counterpart in the reference, whose call
//                       is one table lookup and one launch): microseconds per
//                       rocm_sgemm_find_config, and per enqueued call while the GPU has queue space
//   --mfma_ceiling      what the matrix pipes reach with nothing else to do: a kernel of MFMAs only,
//                       one workgroup per CU, with the shader clock of every XCD during the run
//   --l2_to_lds         bytes per cycle and CU that direct-to-LDS loads deliver from windows that fit
//                       the L2s and from windows that do not
//   --pmc               short run for use under rocprofv3 --pmc: 2 warm-up + 5 timed launches and
//                       one plain 64 MiB copy kernel, whose known traffic calibrates the
//                       FETCH_SIZE / WRITE_SIZE counters

#include <algorithm>
#include <chrono>
#include <filesystem>
#include <fstream>
#include <map>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <limits>
#include <random>
#include <sstream>
#include <string>
#include <thread>
#include <tuple>
#include <vector>

#include <hip/hip_runtime.h>
#include <rocm_sgemm.h>
#include <rocm_sgemm/gemm.hpp>

#include "sampled_check.hpp"

#ifdef BENCH_WITH_ROCBLAS
#include <rocblas/rocblas.h>
#endif
#ifdef BENCH_WITH_HIPBLASLT
#include <hipblaslt/hipblaslt.h>
#endif

namespace
{

using rocm_sgemm::m_layout;

constexpr double peak_tflops = 157.3; // MI355X dense FP32 matrix peak

#define HIP_CHECK(call)                                                                          \
    do                                                                                           \
    {                                                                                            \
        hipError_t status_ = (call);                                                             \
        if(status_ != hipSuccess)                                                                \
        {                                                                                        \
            std::fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(status_), __FILE__, \
                         __LINE__);                                                              \
            std::exit(EXIT_FAILURE);                                                             \
        }                                                                                        \
    } while(0)

struct options
{
    std::vector<std::tuple<size_t, size_t, size_t>> shapes
        = {{1024, 1024, 1024}, {2048, 2048, 2048}, {4096, 4096, 4096}, {8192, 8192, 8192}};
    int              batch_count = 1;
    int              warmup      = 10;
    int              iters       = 100;
    bool             identity_b  = false;
    bool             uniform     = false;
    unsigned         seed        = 0;
    bool             verify      = false;
    int              cpu_threads = -1; // -1: no CPU row
    bool             vendor      = false;
    bool             pmc         = false; // child mode under rocprofv3
    bool             counters    = false; // parent mode: collect counters row by row
    bool             l2_to_lds    = false; // time the L2 -> LDS path alone instead of the timing table
    bool             mfma_ceiling = false; // time the matrix pipes alone instead of the timing table
    bool             host_cost   = false; // host-side cost of a call instead of the timing table
    std::vector<int> layouts; // bit 2 = A col, bit 1 = B col, bit 0 = C col; empty = all eight
};

// Logical (row, column) -> storage index of a dense packed matrix (reference common/matrix.hpp:130-139).
inline size_t at(bool col_major, size_t rows, size_t cols, size_t i, size_t j)
{
    return col_major ? j * rows + i : i * cols + j;
}

// The reference's bench input: a five-value cycle written in logical row-by-row order
// (benchmark/bench.hpp:15-29).
void fill_pattern(std::vector<float>& x, bool col_major, size_t rows, size_t cols)
{
    static const float tmp[5] = {1.025f, 1.05f, 1.075f, 1.1f, 1.0f};
    size_t             l      = 0;
    for(size_t i = 0; i < rows; ++i)
        for(size_t j = 0; j < cols; ++j)
            x[at(col_major, rows, cols, i, j)] = tmp[l++ % 5];
}

void fill_uniform(std::vector<float>& x, bool col_major, size_t rows, size_t cols, std::mt19937& gen)
{
    std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
    for(size_t i = 0; i < rows; ++i)
        for(size_t j = 0; j < cols; ++j)
            x[at(col_major, rows, cols, i, j)] = dist(gen);
}

void fill_identity(std::vector<float>& x, size_t n)
{
    std::fill(x.begin(), x.end(), 0.0f);
    for(size_t i = 0; i < n; ++i)
        x[i * n + i] = 1.0f; // the identity is its own transpose: same image in both layouts
}

std::vector<std::tuple<size_t, size_t, size_t>> parse_shapes(const std::string& text)
{
    std::vector<std::tuple<size_t, size_t, size_t>> shapes;
    std::stringstream                               ss(text);
    std::string                                     token;
    while(std::getline(ss, token, ':'))
    {
        std::vector<size_t> dims;
        std::stringstream   ts(token);
        std::string         dim;
        while(std::getline(ts, dim, ','))
        {
            const size_t b = dim.find_first_not_of(" \t");
            if(b == std::string::npos) continue;
            dims.push_back(std::stoul(dim.substr(b)));
        }
        if(dims.size() == 1)
            shapes.emplace_back(dims[0], dims[0], dims[0]);
        else if(dims.size() == 3)
            shapes.emplace_back(dims[0], dims[1], dims[2]);
        else if(!dims.empty())
            std::cerr << "Warning: Invalid shape format '" << token << "'. Expected 'M' or 'M,N,K'.\n";
    }
    return shapes;
}

void print_usage(const char* program)
{
    std::cout << "Usage: " << program << " [options]\n"
              << "Options:\n"
              << "  --shapes <list>    Colon-separated list of matrix shapes\n"
              << "                     Format: 'M,N,K' for rectangular or 'M' for square (default: "
                 "1024:2048:4096:8192)\n"
              << "  --batch_count <n>  Batch count (default: 1)\n"
              << "  --warmup <n>       untimed launches per benchmark (default: 10)\n"
              << "  --iters <n>        timed launches per benchmark (default: 100)\n"
              << "  --layouts <list>   comma-separated A,B,C layout letters, e.g. rrr,rcr (default: all 8)\n"
              << "  --identity_b       B = identity, output checked bit-exact against A (square shapes)\n"
              << "  --uniform [seed]   uniform[-1,1) inputs from mt19937(seed) instead of the cyclic pattern\n"
              << "  --verify           sampled fp64 check of every result\n"
              << "  --cpu [threads]    also time the reference CPU GEMM on the host (first shape, <= 1024^3)\n"
              << "  --vendor           also time rocBLAS and hipBLASLt (fp32) for context\n"
              << "  --counters         then collect rocprofv3 counters per row: MFMA busy %, LDS conflicts, HBM GB/s\n"
              << "  --pmc              short run (2 warm-up + 5 timed + a copy probe) for use under rocprofv3 --pmc\n"
              << "  --host_cost        host microseconds per call: planning alone, and enqueueing plain / split-K /\n"
              << "                     stream-K-tail products, one shape repeated and several shapes in turn\n"
              << "  --mfma_ceiling     TFLOP/s of a kernel that issues MFMAs only, and the shader clock of every XCD meanwhile\n"
              << "  --l2_to_lds        bytes per cycle and CU of direct-to-LDS loads from L2-resident and larger windows\n"
              << "  --help             Show this help message\n"
              << "\nExamples:\n"
              << "  " << program << " --shapes 512:1024:2048\n"
              << "  " << program << " --shapes 1024,2048,512:2048,1024,1024 --batch_count 4\n";
}

const char* layout_name(bool col)
{
    return col ? "m_layout::col_major" : "m_layout::row_major";
}

// The eight explicit instantiations, selected at run time.
void call_gemm(bool c_col, bool a_col, bool b_col, float* C, float* A, float* B, size_t M, size_t N,
               size_t K, hipStream_t& stream)
{
    constexpr m_layout r = m_layout::row_major, c = m_layout::col_major;
    switch((c_col ? 4 : 0) | (a_col ? 2 : 0) | (b_col ? 1 : 0))
    {
    case 0: rocm_sgemm::gemm<r, r, r>(C, A, B, M, N, K, stream); break;
    case 1: rocm_sgemm::gemm<r, r, c>(C, A, B, M, N, K, stream); break;
    case 2: rocm_sgemm::gemm<r, c, r>(C, A, B, M, N, K, stream); break;
    case 3: rocm_sgemm::gemm<r, c, c>(C, A, B, M, N, K, stream); break;
    case 4: rocm_sgemm::gemm<c, r, r>(C, A, B, M, N, K, stream); break;
    case 5: rocm_sgemm::gemm<c, r, c>(C, A, B, M, N, K, stream); break;
    case 6: rocm_sgemm::gemm<c, c, r>(C, A, B, M, N, K, stream); break;
    default: rocm_sgemm::gemm<c, c, c>(C, A, B, M, N, K, stream); break;
    }
}

struct timing
{
    double avg_ms = 0, min_ms = 0, max_ms = 0, avg_tflops = 0, cpu_ms = 0;
    int    iters = 0;
};

// Warm-up is by count AND by time: after an idle gap the GPU takes tens of milliseconds of
// sustained work to reach its full clock (more for some kernels), so at least `min_warm_ms` of
// back-to-back launches precede the timed ones whatever `warmup` says, continued in batches of
// about 10 ms until two batches in a row agree within 1 % or `max_warm_ms` have passed (0 under
// rocprofv3 --pmc, where every launch is costly).
double min_warm_ms = 40.0;
double max_warm_ms = 600.0;

template<class Launch>
timing time_launches(Launch&& launch, hipStream_t stream, int warmup, int iters, double flops)
{
    hipEvent_t e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    for(int i = 0; i < warmup; ++i)
        launch();
    HIP_CHECK(hipStreamSynchronize(stream));
    double warmed_ms = 0.0, previous = -1.0;
    for(int batch = 4; min_warm_ms > 0.0;)
    {
        HIP_CHECK(hipEventRecord(e0, stream));
        for(int i = 0; i < batch; ++i)
            launch();
        HIP_CHECK(hipEventRecord(e1, stream));
        HIP_CHECK(hipEventSynchronize(e1));
        float ms = 0;
        HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        warmed_ms += ms;
        const double per_launch = (ms > 1e-3f ? ms : 1e-3f) / batch;
        const bool   settled    = previous > 0.0 && std::fabs(per_launch - previous) <= 0.01 * previous;
        previous                = per_launch;
        if(warmed_ms >= min_warm_ms && (settled || warmed_ms >= max_warm_ms)) break;
        const double next = 10.0 / per_launch;
        batch             = next < 2.0 ? 2 : (next > 4096.0 ? 4096 : static_cast<int>(next));
    }
    timing t;
    t.min_ms            = std::numeric_limits<double>::max();
    double sum_ms       = 0, sum_tf = 0;
    const auto wall0    = std::chrono::steady_clock::now();
    for(int i = 0; i < iters; ++i)
    {
        HIP_CHECK(hipEventRecord(e0, stream));
        launch();
        HIP_CHECK(hipPeekAtLastError());
        HIP_CHECK(hipEventRecord(e1, stream));
        HIP_CHECK(hipEventSynchronize(e1));
        float ms = 0;
        HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
        sum_ms += ms;
        sum_tf += flops / (ms * 1e-3) * 1e-12;
        t.min_ms = std::min<double>(t.min_ms, ms);
        t.max_ms = std::max<double>(t.max_ms, ms);
    }
    const auto wall1 = std::chrono::steady_clock::now();
    t.iters          = iters;
    t.avg_ms         = sum_ms / iters;
    t.avg_tflops     = sum_tf / iters;
    t.cpu_ms         = std::chrono::duration<double, std::milli>(wall1 - wall0).count() / iters;
    HIP_CHECK(hipEventDestroy(e0));
    HIP_CHECK(hipEventDestroy(e1));
    return t;
}

void print_header()
{
    const std::string rule(168, '-');
    std::printf("%s\n%-100s %12s %12s %10s %10s %18s %11s %11s %9s\n%s\n", rule.c_str(), "Benchmark",
                "Time", "CPU", "Iterations", "avg_tflops", "bytes_per_second", "max_time_ms",
                "min_time_ms", "pct_peak", rule.c_str());
}

void print_row(const std::string& name, const timing& t, double bytes, const std::string& extra)
{
    const double gib_per_s = bytes / (t.avg_ms * 1e-3) / (1024.0 * 1024.0 * 1024.0);
    std::printf("%-100s %9.3f ms %9.3f ms %10d %10.4f %14.4fGi/s %11.5f %11.5f %9.1f%s\n", name.c_str(),
                t.avg_ms, t.cpu_ms, t.iters, t.avg_tflops, gib_per_s, t.max_ms, t.min_ms,
                100.0 * t.avg_tflops / peak_tflops, extra.c_str());
    std::fflush(stdout);
}

// max |C - C_ref| / (K max|A| max|B|) over 256 sampled entries, C_ref accumulated in fp64; NaN
// when a sampled output is NaN (callers test `err <= tolerance`, which NaN fails)
double sampled_error(const std::vector<float>& C, const std::vector<float>& A, const std::vector<float>& B,
                     size_t M, size_t N, size_t K, bool a_col, bool b_col, bool c_col)
{
    return rocm_sgemm::check::sampled_scaled_error(C.data(), A.data(), B.data(), M, N, K, a_col, b_col, c_col);
}

// The reference's CPU GEMM (test/test.hpp:30-45): i-j-k, fp32 accumulator; rows dealt to threads.
double cpu_gemm_seconds(size_t M, size_t N, size_t K, int threads)
{
    std::vector<float> A(M * K), B(K * N), C(M * N);
    std::mt19937       gen(0);
    fill_uniform(A, false, M, K, gen);
    fill_uniform(B, false, K, N, gen);
    auto body = [&](size_t i0, size_t i1) {
        for(size_t i = i0; i < i1; ++i)
            for(size_t j = 0; j < N; ++j)
            {
                float acc = 0.0f;
                for(size_t k = 0; k < K; ++k)
                    acc += A[i * K + k] * B[k * N + j];
                C[i * N + j] = acc;
            }
    };
    const auto t0 = std::chrono::steady_clock::now();
    if(threads <= 1)
    {
        body(0, M);
    }
    else
    {
        std::vector<std::thread> pool;
        for(int t = 0; t < threads; ++t)
            pool.emplace_back(body, M * t / threads, M * (t + 1) / threads);
        for(auto& th : pool) th.join();
    }
    const auto t1 = std::chrono::steady_clock::now();
    volatile float sink = C[M * N / 2];
    (void)sink;
    return std::chrono::duration<double>(t1 - t0).count();
}

// Plain copy of known size: under rocprofv3 --pmc its FETCH_SIZE / WRITE_SIZE readings give the
// scale of those counters (KiB of HBM traffic per counted unit).
constexpr size_t probe_floats = 16u << 20; // 64 MiB read, 64 MiB written
__global__ void bench_copy_probe(float* __restrict__ dst, const float* __restrict__ src, size_t n)
{
    for(size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n;
        i += static_cast<size_t>(gridDim.x) * blockDim.x)
        dst[i] = src[i];
}

void run_copy_probe()
{
    float *a, *b;
    HIP_CHECK(hipMalloc(&a, probe_floats * sizeof(float)));
    HIP_CHECK(hipMalloc(&b, probe_floats * sizeof(float)));
    HIP_CHECK(hipMemset(a, 0, probe_floats * sizeof(float)));
    for(int i = 0; i < 3; ++i)
        hipLaunchKernelGGL(bench_copy_probe, dim3(4096), dim3(256), 0, nullptr, b, a, probe_floats);
    HIP_CHECK(hipDeviceSynchronize());
    HIP_CHECK(hipFree(a));
    HIP_CHECK(hipFree(b));
}

// ---- the matrix pipes alone ---------------------------------------------------------------------
// One workgroup of four waves per CU (the LDS request keeps a second one out), every wave issuing
// nothing but v_mfma_f32_32x32x2_f32 on four independent accumulator tiles: no loads, no LDS, no
// barriers.  What this reaches is the ceiling any SGEMM kernel on this GPU sample works under; the
// published 157.3 TFLOP/s is 256 CUs x 256 flop per cycle x 2.4 GHz, and the XCDs do not all hold
// 2.4 GHz while their matrix pipes are full.  Each wave records wall-clock (100 MHz) and shader
// clock stamps around its loop, which gives the shader clock of every XCD during the run.
constexpr int burn_lds_floats = 33 * 1024; // 132 KB of the CU's 160 KB
__global__ __launch_bounds__(256) void bench_mfma_burn(unsigned long long* __restrict__ stamps, float* __restrict__ sink,
                                                       int iters)
{
    typedef float f32x16 __attribute__((ext_vector_type(16)));
    __shared__ float pad[burn_lds_floats];
    pad[threadIdx.x] = static_cast<float>(threadIdx.x);
    __syncthreads();
    const float a = pad[(threadIdx.x * 7) % 256] * 1e-4f + 1.0f;
    const float b = pad[(threadIdx.x * 13) % 256] * 1e-4f - 1.0f;
    f32x16      acc[4];
    for(int j = 0; j < 4; ++j)
        for(int v = 0; v < 16; ++v)
            acc[j][v] = 0.0f;
#if defined(__HIP_DEVICE_COMPILE__)
    const unsigned long long t0 = wall_clock64(), c0 = clock64();
    for(int i = 0; i < iters; ++i)
    {
#pragma unroll
        for(int j = 0; j < 4; ++j)
            acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j], 0, 0, 0);
    }
    const unsigned long long t1 = wall_clock64(), c1 = clock64();
    float                    s  = 0.0f;
    for(int j = 0; j < 4; ++j)
        for(int v = 0; v < 16; ++v)
            s += acc[j][v];
    if(s == 0.123456f) sink[0] = s; // keeps the accumulators alive
    if(threadIdx.x % 64 == 0)
    {
        unsigned long long* o = stamps + (static_cast<size_t>(blockIdx.x) * 4 + threadIdx.x / 64) * 4;
        o[0]                  = t0;
        o[1]                  = t1;
        o[2]                  = c1 - c0;
        o[3]                  = __builtin_amdgcn_s_getreg((31 << 11) | 20) & 7; // XCC_ID
    }
#endif
}

int run_mfma_ceiling()
{
    hipDeviceProp_t prop;
    HIP_CHECK(hipGetDeviceProperties(&prop, 0));
    const int           cus = prop.multiProcessorCount, waves = cus * 4;
    unsigned long long* stamps;
    float*              sink;
    HIP_CHECK(hipMalloc(&stamps, sizeof(unsigned long long) * waves * 4));
    HIP_CHECK(hipMalloc(&sink, sizeof(float)));
    const int    iters = 40000; // 160 000 MFMAs per wave: about 4.3 ms
    const double flop  = static_cast<double>(waves) * iters * 4.0 * (2.0 * 32 * 32 * 2);
    hipEvent_t   e0, e1;
    HIP_CHECK(hipEventCreate(&e0));
    HIP_CHECK(hipEventCreate(&e1));
    for(int i = 0; i < 30; ++i) // warm-up: well over 100 ms of sustained work
        hipLaunchKernelGGL(bench_mfma_burn, dim3(cus), dim3(256), 0, nullptr, stamps, sink, iters);
    HIP_CHECK(hipEventRecord(e0, nullptr));
    const int launches = 10;
    for(int i = 0; i < launches; ++i)
        hipLaunchKernelGGL(bench_mfma_burn, dim3(cus), dim3(256), 0, nullptr, stamps, sink, iters);
    HIP_CHECK(hipEventRecord(e1, nullptr));
    HIP_CHECK(hipEventSynchronize(e1));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::vector<unsigned long long> h(static_cast<size_t>(waves) * 4);
    HIP_CHECK(hipMemcpy(h.data(), stamps, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    std::printf("mfma_ceiling  %d CUs x 4 waves, %d v_mfma_f32_32x32x2_f32 per wave and launch, %d launches back to back\n",
                cus, iters * 4, launches);
    std::printf("mfma_ceiling  whole launches (event pair around all of them): %.3f ms each = %.1f TFLOP/s = %.1f %% of %.1f\n",
                ms / launches, flop / (ms / launches) * 1e-9, flop / (ms / launches) * 1e-9 / (cus * 256 * 2.4e-3) * 100.0,
                cus * 256 * 2.4e-3);
    double mhz[8] = {0}, us[8] = {0};
    int    count[8] = {0};
    for(int w = 0; w < waves; ++w)
    {
        const unsigned long long* o = &h[static_cast<size_t>(w) * 4];
        const int                 x = static_cast<int>(o[3]);
        mhz[x] += static_cast<double>(o[2]) / static_cast<double>(o[1] - o[0]) * 100.0;
        us[x] += static_cast<double>(o[1] - o[0]) * 0.01;
        count[x]++;
    }
    double slowest = 0, mean = 0;
    int    xcds = 0;
    for(int x = 0; x < 8; ++x)
        if(count[x] > 0)
        {
            std::printf("mfma_ceiling  XCD %d: %4d waves, shader clock %.0f MHz, loop %.1f us = %.1f %% of the matrix pipes' %d cycles\n",
                        x, count[x], mhz[x] / count[x], us[x] / count[x],
                        iters * 4.0 * 64.0 / (mhz[x] / count[x] * us[x] / count[x]) * 100.0, iters * 4 * 64);
            slowest = std::max(slowest, us[x] / count[x]);
            mean += us[x] / count[x];
            ++xcds;
        }
    std::printf("mfma_ceiling  by the slowest XCD's loop: %.1f TFLOP/s; by the mean over XCDs: %.1f TFLOP/s\n",
                flop / slowest * 1e-6, flop / (mean / xcds) * 1e-6);
    HIP_CHECK(hipFree(stamps));
    HIP_CHECK(hipFree(sink));
    return 0;
}

// ---- the path from L2 into LDS alone ----------------------------------------------------------------
// Every workgroup (256 threads, one per CU) streams 16-byte pieces straight into LDS
// (buffer_load_dwordx4 ... lds, the instruction the GEMM kernels move their operands with) from a
// window of its own that it reads over and over: a window larger than the CU's vector cache and
// small enough for all windows to stay in the L2s measures L2 -> LDS; a larger one measures what
// comes from beyond the L2.  The figure bounds the operand traffic a GEMM kernel can ask of a CU.
template<int WINDOW_KB>
__global__ __launch_bounds__(256) void bench_l2_to_lds(const float* __restrict__ src, float* __restrict__ sink,
                                                       unsigned long long* __restrict__ cycles, int iters)
{
    __shared__ __attribute__((aligned(16))) float lds[4 * 1024]; // 16 KB: four loads of the workgroup
#if defined(__HIP_DEVICE_COMPILE__)
    const float* base = src + static_cast<size_t>(blockIdx.x) * WINDOW_KB * 256;
    const __amdgpu_buffer_rsrc_t rsrc
        = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, WINDOW_KB * 1024, 0x00020000);
    const int                wave = threadIdx.x / 64;
    const unsigned long long c0   = clock64();
    for(int i = 0; i < iters; ++i)
    {
#pragma unroll
        for(int u = 0; u < 4; ++u) // 4 KB per load of the workgroup
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)(lds + (u * 256 + wave * 64) * 4),
                                                     16, threadIdx.x * 16, ((i * 4 + u) % (WINDOW_KB / 4)) * 4096, 0, 0);
        if((i & 7) == 7) __builtin_amdgcn_s_waitcnt(0x0070 | 8); // at most eight loads of the wave in flight
    }
    __builtin_amdgcn_s_waitcnt(0);
    const unsigned long long c1 = clock64();
    if(lds[threadIdx.x] == 0.12345f) sink[0] = lds[threadIdx.x];
    if(threadIdx.x == 0) cycles[blockIdx.x] = c1 - c0;
#else
    (void)src, (void)sink, (void)cycles, (void)iters, (void)lds;
#endif
}

template<int WINDOW_KB>
int run_l2_to_lds_case(int groups, const float* src, float* sink, unsigned long long* cycles)
{
    const int iters = 4000; // 64 MB per workgroup
    for(int r = 0; r < 3; ++r)
        hipLaunchKernelGGL(bench_l2_to_lds<WINDOW_KB>, dim3(groups), dim3(256), 0, nullptr, src, sink, cycles, iters);
    HIP_CHECK(hipDeviceSynchronize());
    std::vector<unsigned long long> h(groups);
    HIP_CHECK(hipMemcpy(h.data(), cycles, groups * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    double mean = 0;
    for(unsigned long long v : h)
        mean += static_cast<double>(v);
    mean /= groups;
    const double per_cu = iters * 16384.0 / mean;
    std::printf("l2_to_lds  window %4d KB per workgroup, %3d workgroups (%5.1f MB in all): %5.1f bytes per cycle and CU = %5.1f TB/s at 2.4 GHz\n",
                WINDOW_KB, groups, groups * WINDOW_KB / 1024.0, per_cu, per_cu * groups * 2.4e-3);
    return 0;
}

int run_l2_to_lds()
{
    float *            src, *sink;
    unsigned long long* cycles;
    HIP_CHECK(hipMalloc(&src, 256u << 20));
    HIP_CHECK(hipMemset(src, 0, 256u << 20));
    HIP_CHECK(hipMalloc(&sink, sizeof(float)));
    HIP_CHECK(hipMalloc(&cycles, 1024 * sizeof(unsigned long long)));
    hipDeviceProp_t prop;
    HIP_CHECK(hipGetDeviceProperties(&prop, 0));
    const int cus = prop.multiProcessorCount;
    for(int groups : {cus / 4, cus})
    {
        run_l2_to_lds_case<64>(groups, src, sink, cycles);
        run_l2_to_lds_case<128>(groups, src, sink, cycles);
        run_l2_to_lds_case<256>(groups, src, sink, cycles);
        run_l2_to_lds_case<1024>(groups, src, sink, cycles);
    }
    HIP_CHECK(hipFree(src));
    HIP_CHECK(hipFree(sink));
    HIP_CHECK(hipFree(cycles));
    return 0;
}

// ---- counters: parent side ------------------------------------------------------------------------

struct counter_pass
{
    const char* name;
    const char* counters;
};
const counter_pass counter_passes[] = {
    {"mfma", "SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CU_CYCLES GRBM_GUI_ACTIVE SQ_INSTS_VALU_MFMA_MOPS_F32"},
    {"lds", "SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE"},
    {"fetch", "FETCH_SIZE"},
    {"write", "WRITE_SIZE"},
};

// Splits one CSV line, honouring double quotes (kernel names contain commas).
std::vector<std::string> split_csv(const std::string& line)
{
    std::vector<std::string> out;
    std::string              cur;
    bool                     quoted = false;
    for(char ch : line)
    {
        if(ch == '"')
            quoted = !quoted;
        else if(ch == ',' && !quoted)
        {
            out.push_back(cur);
            cur.clear();
        }
        else
            cur.push_back(ch);
    }
    out.push_back(cur);
    return out;
}

// Mean per-dispatch value of every counter, for the GEMM kernel ("gemm:<counter>") and for the
// copy probe ("copy:<counter>"), from the counter_collection CSV files rocprofv3 left under `dir`.
std::map<std::string, double> read_counters(const std::string& dir)
{
    std::map<std::string, std::pair<double, int>> acc;
    namespace fs = std::filesystem;
    std::error_code ec;
    for(fs::recursive_directory_iterator it(dir, ec), end; !ec && it != end; it.increment(ec))
    {
        const std::string path = it->path().string();
        if(path.find("counter_collection.csv") == std::string::npos) continue;
        std::ifstream in(path);
        std::string   line;
        if(!std::getline(in, line)) continue;
        const std::vector<std::string> head = split_csv(line);
        int                            c_kernel = -1, c_name = -1, c_value = -1;
        for(size_t i = 0; i < head.size(); ++i)
        {
            if(head[i] == "Kernel_Name") c_kernel = static_cast<int>(i);
            if(head[i] == "Counter_Name") c_name = static_cast<int>(i);
            if(head[i] == "Counter_Value") c_value = static_cast<int>(i);
        }
        if(c_kernel < 0 || c_name < 0 || c_value < 0) continue;
        while(std::getline(in, line))
        {
            const std::vector<std::string> f = split_csv(line);
            if(static_cast<int>(f.size()) <= std::max(c_kernel, std::max(c_name, c_value))) continue;
            const char* tag = f[c_kernel].find("sgemm_mfma_kernel") != std::string::npos
                                  ? "gemm:"
                                  : (f[c_kernel].find("bench_copy_probe") != std::string::npos ? "copy:" : nullptr);
            if(tag == nullptr) continue;
            auto& slot = acc[std::string(tag) + f[c_name]];
            slot.first += std::atof(f[c_value].c_str());
            slot.second += 1;
        }
    }
    std::map<std::string, double> out;
    for(const auto& kv : acc)
        out[kv.first] = kv.second.first / kv.second.second;
    return out;
}

std::string shell_quote(const std::string& s)
{
    std::string out = "'";
    for(char ch : s)
        out += ch == '\'' ? std::string("'\\''") : std::string(1, ch);
    return out + "'";
}

// Runs this program (one shape, one layout combination, --pmc) under rocprofv3 once per counter
// set and prints the derived figures.  Nothing here touches the GPU.
int collect_counters(const options& opt, const char* self)
{
    namespace fs = std::filesystem;
    std::error_code ec;
    const std::string exe = fs::canonical(self, ec).string();
    if(ec || std::system("command -v rocprofv3 > /dev/null 2>&1") != 0)
    {
        std::fprintf(stderr, "--counters needs rocprofv3 on PATH and a resolvable program path\n");
        return 2;
    }
    std::printf("\nhardware counters (rocprofv3 --pmc, mean per launch of the GEMM kernel; HBM bytes scaled by a 64 MiB copy probe)\n");
    std::printf("mfma_busy_pct: matrix-pipe busy cycles over the GPU's active cycles, which under the profiler include about\n"
                "10 us of dispatch overhead per launch; of_cu_busy: over the cycles in which the CUs hold waves of the kernel\n");
    std::printf("%-100s %13s %10s %20s %16s %12s\n", "Benchmark", "mfma_busy_pct", "of_cu_busy", "lds_bank_conflict_pct",
                "hbm_MB_per_launch", "hbm_GBps");
    int failures = 0;
    for(const auto& shape : opt.shapes)
    {
        const size_t M = std::get<0>(shape), N = std::get<1>(shape), K = std::get<2>(shape);
        for(int c_col = 1; c_col >= 0; --c_col)
            for(int b_col = 1; b_col >= 0; --b_col)
                for(int a_col = 1; a_col >= 0; --a_col)
                {
                    const int code = (a_col << 2) | (b_col << 1) | c_col;
                    if(!opt.layouts.empty()
                       && std::find(opt.layouts.begin(), opt.layouts.end(), code) == opt.layouts.end())
                        continue;
                    const std::string lay = std::string(a_col ? "c" : "r") + (b_col ? "c" : "r") + (c_col ? "c" : "r");
                    std::map<std::string, double> all;
                    double                        avg_ms = 0;
                    for(const counter_pass& pass : counter_passes)
                    {
                        char tmpl[] = "/tmp/bench_float_pmc_XXXXXX";
                        if(mkdtemp(tmpl) == nullptr) return 2;
                        const std::string dir = tmpl;
                        const std::string cmd
                            = "cd /tmp && TMPDIR=/tmp rocprofv3 --pmc " + std::string(pass.counters)
                              + " --output-format csv -d " + shell_quote(dir) + " -- " + shell_quote(exe)
                              + " --pmc --shapes " + std::to_string(M) + "," + std::to_string(N) + ","
                              + std::to_string(K) + " --layouts " + lay
                              + (opt.identity_b ? " --identity_b" : (opt.uniform ? " --uniform" : ""))
                              + " > " + shell_quote(dir + "/stdout.txt") + " 2> /dev/null";
                        const int rc = std::system(cmd.c_str());
                        if(rc != 0)
                        {
                            std::fprintf(stderr, "counter pass %s failed (exit %d)\n", pass.name, rc);
                            ++failures;
                        }
                        for(const auto& kv : read_counters(dir))
                            all[kv.first] = kv.second;
                        // the child's own timing row: "... }/manual_time  <avg> ms ..."
                        std::ifstream in(dir + "/stdout.txt");
                        std::string   line;
                        while(std::getline(in, line))
                        {
                            const size_t at_ = line.find("}/manual_time");
                            if(at_ != std::string::npos && line.compare(0, 3, "{A:") == 0)
                                avg_ms = std::atof(line.c_str() + at_ + 13);
                        }
                        fs::remove_all(dir, ec);
                    }
                    const std::string name = std::string("{A:") + layout_name(a_col) + ",B:" + layout_name(b_col)
                                             + ",C:" + layout_name(c_col) + ",m:" + std::to_string(M) + ",n:"
                                             + std::to_string(N) + ",k:" + std::to_string(K) + "}/counters";
                    // GRBM_GUI_ACTIVE is summed over the 8 XCDs, MFMA busy cycles over the 4 SIMDs of each CU
                    const double simds = 4.0 * 256.0;
                    const double busy = all.count("gemm:SQ_VALU_MFMA_BUSY_CYCLES") && all["gemm:GRBM_GUI_ACTIVE"] > 0
                                            ? 100.0 * all["gemm:SQ_VALU_MFMA_BUSY_CYCLES"]
                                                  / (all["gemm:GRBM_GUI_ACTIVE"] / 8.0 * simds)
                                            : -1.0;
                    // SQ_BUSY_CU_CYCLES: summed over the CUs, cycles in which a CU holds at least one wave
                    const double busy_cu = all.count("gemm:SQ_VALU_MFMA_BUSY_CYCLES") && all["gemm:SQ_BUSY_CU_CYCLES"] > 0
                                               ? 100.0 * all["gemm:SQ_VALU_MFMA_BUSY_CYCLES"]
                                                     / (all["gemm:SQ_BUSY_CU_CYCLES"] * 4.0)
                                               : -1.0;
                    const double conf = all.count("gemm:SQ_LDS_BANK_CONFLICT") && all["gemm:SQ_LDS_IDX_ACTIVE"] > 0
                                            ? 100.0 * all["gemm:SQ_LDS_BANK_CONFLICT"] / all["gemm:SQ_LDS_IDX_ACTIVE"]
                                            : -1.0;
                    const double probe_kib = probe_floats * sizeof(float) / 1024.0;
                    const double f_scale = all["copy:FETCH_SIZE"] > 0 ? probe_kib / all["copy:FETCH_SIZE"] : 1.0;
                    const double w_scale = all["copy:WRITE_SIZE"] > 0 ? probe_kib / all["copy:WRITE_SIZE"] : 1.0;
                    const double bytes = (all["gemm:FETCH_SIZE"] * f_scale + all["gemm:WRITE_SIZE"] * w_scale) * 1024.0;
                    std::printf("%-100s %13.2f %10.2f %20.2f %16.1f %12.1f\n", name.c_str(), busy, busy_cu, conf, bytes * 1e-6,
                                avg_ms > 0 ? bytes / (avg_ms * 1e-3) * 1e-9 : -1.0);
                    std::fflush(stdout);
                }
    }
    return failures == 0 ? 0 : 1;
}

// A vendor BLAS computes a column-major D(m x n) = op(X) op(Y).  Column-major C is the product as
// it stands (X = A, Y = B; a row-major operand is the transpose of a column-major one, reference
// rocblas_wrapper/src/gemm.cpp:45-58); row-major C (M x N) is the column-major N x M matrix
// C^T = B^T A^T, so the operands swap and the transposition flags flip.
struct vendor_problem
{
    bool         trans_x, trans_y;
    int          m, n, k, ldx, ldy, ldd;
    const float *x, *y;
};

vendor_problem vendor_map(bool a_col, bool b_col, bool c_col, size_t M, size_t N, size_t K,
                          const float* A, const float* B)
{
    vendor_problem p;
    p.k = static_cast<int>(K);
    if(c_col)
    {
        p.m = static_cast<int>(M), p.n = static_cast<int>(N);
        p.x = A, p.trans_x = !a_col, p.ldx = static_cast<int>(a_col ? M : K);
        p.y = B, p.trans_y = !b_col, p.ldy = static_cast<int>(b_col ? K : N);
    }
    else
    {
        p.m = static_cast<int>(N), p.n = static_cast<int>(M);
        p.x = B, p.trans_x = b_col, p.ldx = static_cast<int>(b_col ? K : N);
        p.y = A, p.trans_y = a_col, p.ldy = static_cast<int>(a_col ? M : K);
    }
    p.ldd = p.m;
    return p;
}

#ifdef BENCH_WITH_HIPBLASLT
// One hipBLASLt fp32 matmul plan (descriptor, layouts, the heuristic's first algorithm, workspace).
struct lt_plan
{
    hipblasLtHandle_t       handle = nullptr;
    hipblasLtMatmulDesc_t   desc   = nullptr;
    hipblasLtMatrixLayout_t lx = nullptr, ly = nullptr, ld = nullptr;
    hipblasLtMatmulAlgo_t   algo{};
    void*                   workspace      = nullptr;
    size_t                  workspace_size = 0;
    bool                    ok             = false;

    lt_plan(hipblasLtHandle_t h, const vendor_problem& p) : handle(h)
    {
        const size_t max_ws = size_t(64) << 20;
        if(hipblasLtMatmulDescCreate(&desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return;
        const hipblasOperation_t ox = p.trans_x ? HIPBLAS_OP_T : HIPBLAS_OP_N;
        const hipblasOperation_t oy = p.trans_y ? HIPBLAS_OP_T : HIPBLAS_OP_N;
        hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSA, &ox, sizeof(ox));
        hipblasLtMatmulDescSetAttribute(desc, HIPBLASLT_MATMUL_DESC_TRANSB, &oy, sizeof(oy));
        // stored shapes: an operand used transposed is held as (k x m) / (n x k)
        if(hipblasLtMatrixLayoutCreate(&lx, HIP_R_32F, p.trans_x ? p.k : p.m, p.trans_x ? p.m : p.k, p.ldx)
               != HIPBLAS_STATUS_SUCCESS
           || hipblasLtMatrixLayoutCreate(&ly, HIP_R_32F, p.trans_y ? p.n : p.k, p.trans_y ? p.k : p.n, p.ldy)
                  != HIPBLAS_STATUS_SUCCESS
           || hipblasLtMatrixLayoutCreate(&ld, HIP_R_32F, p.m, p.n, p.ldd) != HIPBLAS_STATUS_SUCCESS)
            return;
        hipblasLtMatmulPreference_t pref = nullptr;
        if(hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return;
        hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &max_ws,
                                              sizeof(max_ws));
        hipblasLtMatmulHeuristicResult_t result[1];
        int                              found = 0;
        const hipblasStatus_t st = hipblasLtMatmulAlgoGetHeuristic(handle, desc, lx, ly, ld, ld, pref, 1,
                                                                   result, &found);
        hipblasLtMatmulPreferenceDestroy(pref);
        if(st != HIPBLAS_STATUS_SUCCESS || found < 1) return;
        algo           = result[0].algo;
        workspace_size = result[0].workspaceSize;
        if(workspace_size > 0 && hipMalloc(&workspace, workspace_size) != hipSuccess) return;
        ok = true;
    }
    lt_plan(const lt_plan&)            = delete;
    lt_plan& operator=(const lt_plan&) = delete;
    ~lt_plan()
    {
        if(workspace) (void)hipFree(workspace);
        if(ld) hipblasLtMatrixLayoutDestroy(ld);
        if(ly) hipblasLtMatrixLayoutDestroy(ly);
        if(lx) hipblasLtMatrixLayoutDestroy(lx);
        if(desc) hipblasLtMatmulDescDestroy(desc);
    }
    hipblasStatus_t run(const vendor_problem& p, float* D, hipStream_t stream) const
    {
        const float one = 1.0f, zero = 0.0f;
        return hipblasLtMatmul(handle, desc, &one, p.x, lx, p.y, ly, &zero, D, ld, D, ld, &algo, workspace,
                               workspace_size, stream);
    }
};
#endif

int run(const options& opt)
{
    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
#ifdef BENCH_WITH_ROCBLAS
    rocblas_handle handle = nullptr;
    if(opt.vendor)
    {
        if(rocblas_create_handle(&handle) != rocblas_status_success
           || rocblas_set_stream(handle, stream) != rocblas_status_success)
        {
            std::fprintf(stderr, "rocBLAS initialisation failed\n");
            return 1;
        }
    }
#endif
#ifdef BENCH_WITH_HIPBLASLT
    hipblasLtHandle_t lt_handle = nullptr;
    if(opt.vendor && hipblasLtCreate(&lt_handle) != HIPBLAS_STATUS_SUCCESS)
    {
        std::fprintf(stderr, "hipBLASLt initialisation failed\n");
        return 1;
    }
#endif
    hipDeviceProp_t prop;
    HIP_CHECK(hipGetDeviceProperties(&prop, 0));
    std::printf("device: %s %s, %d CUs, %d MHz; peak used for pct_peak: %.1f TFLOP/s (dense FP32 matrix)\n",
                prop.name, prop.gcnArchName, prop.multiProcessorCount, prop.clockRate / 1000, peak_tflops);
    std::printf("protocol: %d warm-up launches (and at least %.0f ms of them, until the launch time has settled) + %d "
                "timed launches per row, one event pair per launch, each waited for; inputs: %s\n",
                opt.warmup, min_warm_ms, opt.iters,
                opt.identity_b ? "A uniform[-1,1), B = identity"
                               : (opt.uniform ? "uniform[-1,1)" : "cyclic {1.025,1.05,1.075,1.1,1.0}"));
    print_header();

    int failures = 0;
    for(const auto& shape : opt.shapes)
    {
        const size_t M = std::get<0>(shape), N = std::get<1>(shape), K = std::get<2>(shape);
        if(opt.identity_b && N != K)
        {
            std::fprintf(stderr, "--identity_b needs N == K; skipping %zux%zux%zu\n", M, N, K);
            continue;
        }
        // layout combinations in the reference's registration order (bench.cpp:240-303):
        // C column-major first, then (A,B) = cc, rc, cr, rr
        std::vector<std::tuple<bool, bool, bool>> combos;
        for(int c_col = 1; c_col >= 0; --c_col)
            for(int b_col = 1; b_col >= 0; --b_col)
                for(int a_col = 1; a_col >= 0; --a_col)
                {
                    const int code = (a_col << 2) | (b_col << 1) | c_col;
                    if(opt.layouts.empty()
                       || std::find(opt.layouts.begin(), opt.layouts.end(), code) != opt.layouts.end())
                        combos.emplace_back(a_col != 0, b_col != 0, c_col != 0);
                }
        const size_t batch = static_cast<size_t>(opt.batch_count);
        for(const auto& combo : combos)
        {
            const bool a_col = std::get<0>(combo), b_col = std::get<1>(combo), c_col = std::get<2>(combo);
            std::vector<float> hA(M * K), hB(K * N), hC(M * N);
            if(opt.identity_b || opt.uniform)
            {
                std::mt19937 gen(opt.seed);
                fill_uniform(hA, a_col, M, K, gen);
                if(opt.identity_b)
                    fill_identity(hB, K);
                else
                    fill_uniform(hB, b_col, K, N, gen);
            }
            else
            {
                fill_pattern(hA, a_col, M, K);
                fill_pattern(hB, b_col, K, N);
            }
            float *dA, *dB, *dC;
            HIP_CHECK(hipMalloc(&dA, hA.size() * batch * sizeof(float)));
            HIP_CHECK(hipMalloc(&dB, hB.size() * batch * sizeof(float)));
            HIP_CHECK(hipMalloc(&dC, hC.size() * batch * sizeof(float)));
            // as in the reference, batch_count only scales the buffers and the flop count; one
            // product is launched on batch 0 (bench.cpp:49-51,72,77-85)
            for(size_t b = 0; b < batch; ++b)
            {
                HIP_CHECK(hipMemcpy(dA + b * hA.size(), hA.data(), hA.size() * sizeof(float), hipMemcpyHostToDevice));
                HIP_CHECK(hipMemcpy(dB + b * hB.size(), hB.data(), hB.size() * sizeof(float), hipMemcpyHostToDevice));
            }
            HIP_CHECK(hipMemset(dC, 0xFF, hC.size() * sizeof(float)));
            HIP_CHECK(hipDeviceSynchronize());

            const double flops = 2.0 * M * N * K * batch;
            const double bytes = static_cast<double>(M * K + K * N + M * N) * sizeof(float);
            const timing t     = time_launches(
                [&] { call_gemm(c_col, a_col, b_col, dC, dA, dB, M, N, K, stream); }, stream,
                opt.warmup, opt.iters, flops);

            std::string extra;
            if(opt.identity_b || opt.verify)
            {
                HIP_CHECK(hipMemcpy(hC.data(), dC, hC.size() * sizeof(float), hipMemcpyDeviceToHost));
                if(opt.identity_b)
                {
                    // C (M x N, layout c) must hold A (M x K = M x N, layout a) bit for bit
                    size_t bad = 0;
                    for(size_t i = 0; i < M && bad == 0; ++i)
                        for(size_t j = 0; j < N; ++j)
                        {
                            const float got = hC[at(c_col, M, N, i, j)], want = hA[at(a_col, M, K, i, j)];
                            if(std::memcmp(&got, &want, sizeof(float)) != 0)
                            {
                                ++bad;
                                break;
                            }
                        }
                    extra += bad ? "  identity:MISMATCH" : "  identity:bit-exact";
                    failures += bad ? 1 : 0;
                }
                if(opt.verify)
                {
                    const double err = sampled_error(hC, hA, hB, M, N, K, a_col, b_col, c_col);
                    char         buf[64];
                    std::snprintf(buf, sizeof(buf), "  err:%.2e%s", err, err <= 1e-6 ? "" : "(FAIL)");
                    extra += buf;
                    failures += err <= 1e-6 ? 0 : 1;
                }
            }
            std::string name = std::string("{A:") + layout_name(a_col) + ",B:" + layout_name(b_col)
                               + ",C:" + layout_name(c_col) + ",m:" + std::to_string(M) + ",n:"
                               + std::to_string(N) + ",k:" + std::to_string(K) + "}/manual_time";
            print_row(name, t, bytes, extra);

            // vendor rows for context; when --verify is given their result is checked the same way
            const auto vendor_row = [&](const std::string& label, const timing& v) {
                std::string note;
                if(opt.verify)
                {
                    HIP_CHECK(hipMemcpy(hC.data(), dC, hC.size() * sizeof(float), hipMemcpyDeviceToHost));
                    const double err = sampled_error(hC, hA, hB, M, N, K, a_col, b_col, c_col);
                    char         buf[64];
                    std::snprintf(buf, sizeof(buf), "  err:%.2e", err);
                    note = buf;
                }
                print_row("  " + label + " " + name, v, bytes, note);
            };
#ifdef BENCH_WITH_ROCBLAS
            if(opt.vendor)
            {
                const vendor_problem p   = vendor_map(a_col, b_col, c_col, M, N, K, dA, dB);
                const float          one = 1.0f, zero = 0.0f;
                HIP_CHECK(hipMemsetAsync(dC, 0xFF, hC.size() * sizeof(float), stream));
                const timing v = time_launches(
                    [&] {
                        rocblas_sgemm(handle, p.trans_x ? rocblas_operation_transpose : rocblas_operation_none,
                                      p.trans_y ? rocblas_operation_transpose : rocblas_operation_none, p.m, p.n,
                                      p.k, &one, p.x, p.ldx, p.y, p.ldy, &zero, dC, p.ldd);
                    },
                    stream, opt.warmup, opt.iters, flops);
                vendor_row("rocBLAS", v);
            }
#endif
#ifdef BENCH_WITH_HIPBLASLT
            if(opt.vendor)
            {
                const vendor_problem p = vendor_map(a_col, b_col, c_col, M, N, K, dA, dB);
                const lt_plan        plan(lt_handle, p);
                if(!plan.ok)
                    std::printf("  hipBLASLt %s: no algorithm\n", name.c_str());
                else
                {
                    HIP_CHECK(hipMemsetAsync(dC, 0xFF, hC.size() * sizeof(float), stream));
                    bool         failed = false;
                    const timing v      = time_launches(
                        [&] { failed |= plan.run(p, dC, stream) != HIPBLAS_STATUS_SUCCESS; }, stream,
                        opt.warmup, opt.iters, flops);
                    if(failed)
                        std::printf("  hipBLASLt %s: hipblasLtMatmul failed\n", name.c_str());
                    else
                        vendor_row("hipBLASLt", v);
                }
            }
#endif
            HIP_CHECK(hipFree(dA));
            HIP_CHECK(hipFree(dB));
            HIP_CHECK(hipFree(dC));
        }
    }

    if(opt.cpu_threads >= 0 && !opt.shapes.empty())
    {
        const size_t M = std::min<size_t>(std::get<0>(opt.shapes[0]), 1024);
        const size_t N = std::min<size_t>(std::get<1>(opt.shapes[0]), 1024);
        const size_t K = std::min<size_t>(std::get<2>(opt.shapes[0]), 1024);
        const int    hw      = static_cast<int>(std::thread::hardware_concurrency());
        const int    threads = opt.cpu_threads == 0 ? std::max(1, hw) : opt.cpu_threads;
        const double s1      = cpu_gemm_seconds(M, N, K, 1);
        std::printf("cpu_reference_gemm{m:%zu,n:%zu,k:%zu,threads:1}  %.3f s  %.6f TFLOP/s\n", M, N, K, s1,
                    2.0 * M * N * K / s1 * 1e-12);
        if(threads > 1)
        {
            const double sn = cpu_gemm_seconds(M, N, K, threads);
            std::printf("cpu_reference_gemm{m:%zu,n:%zu,k:%zu,threads:%d}  %.3f s  %.6f TFLOP/s\n", M, N, K,
                        threads, sn, 2.0 * M * N * K / sn * 1e-12);
        }
    }
#ifdef BENCH_WITH_ROCBLAS
    if(handle != nullptr) rocblas_destroy_handle(handle);
#endif
#ifdef BENCH_WITH_HIPBLASLT
    if(lt_handle != nullptr) hipblasLtDestroy(lt_handle);
#endif
    if(opt.pmc) run_copy_probe();
    HIP_CHECK(hipStreamDestroy(stream));
    return failures == 0 ? 0 : 1;
}

// Host-side cost of a call.  Planning is timed on its own (host only, runs without a GPU); the
// whole call is timed as the mean host time to enqueue a burst of calls that is short enough for
// the GPU queue never to fill, so the host is never waiting for the device.
int run_host_cost()
{
    using clock = std::chrono::steady_clock;
    struct shape
    {
        size_t m, n, k;
    };
    const auto us_per = [](clock::time_point t0, clock::time_point t1, int n) {
        return std::chrono::duration<double, std::micro>(t1 - t0).count() / n;
    };
    const auto plan_cost = [&](const char* what, const std::vector<shape>& shapes) {
        rocm_sgemm_config cfg;
        const int         n  = 200000;
        const auto        t0 = clock::now();
        for(int i = 0; i < n; ++i)
        {
            const shape& s = shapes[i % shapes.size()];
            rocm_sgemm_find_config(s.m, s.n, s.k, 0, 0, 0, &cfg);
        }
        std::printf("host_cost plan  %-58s %8.3f us per call\n", what, us_per(t0, clock::now(), n));
    };
    plan_cost("table entry (4096^3)", {{4096, 4096, 4096}});
    plan_cost("planned shape, repeated (1536 x 1200 x 900)", {{1536, 1200, 900}});
    plan_cost("two planned shapes in turn", {{1536, 1200, 900}, {777, 2222, 1111}});
    plan_cost("six planned shapes in turn",
              {{1536, 1200, 900}, {777, 2222, 1111}, {640, 640, 3000}, {3000, 200, 500}, {96, 5000, 800}, {2100, 2100, 2100}});
    std::vector<shape> many;
    for(size_t i = 0; i < 20; ++i) many.push_back({1500 + 37 * i, 900 + 101 * i, 700 + 53 * i});
    plan_cost("twenty planned shapes in turn (a thread remembers sixteen)", many);

    int devices = 0;
    if(hipGetDeviceCount(&devices) != hipSuccess || devices == 0)
    {
        (void)hipGetLastError();
        std::printf("host_cost call  (no GPU visible: call rows skipped)\n");
        return 0;
    }
    hipStream_t stream;
    HIP_CHECK(hipStreamCreate(&stream));
    const size_t       big = 4096 * 4096;
    float *            dA, *dB, *dC;
    HIP_CHECK(hipMalloc(&dA, big * sizeof(float)));
    HIP_CHECK(hipMalloc(&dB, big * sizeof(float)));
    HIP_CHECK(hipMalloc(&dC, big * sizeof(float)));
    HIP_CHECK(hipMemset(dA, 0, big * sizeof(float)));
    HIP_CHECK(hipMemset(dB, 0, big * sizeof(float)));
    const auto call_cost = [&](const char* what, const std::vector<shape>& shapes) {
        const int burst = 64, rounds = 20;
        for(const shape& s : shapes) // first calls: kernels loaded, workspace of the stream in place
            rocm_sgemm_f32(0, 0, 0, dC, dA, dB, s.m, s.n, s.k, stream);
        HIP_CHECK(hipStreamSynchronize(stream));
        double total = 0.0;
        for(int r = 0; r < rounds; ++r)
        {
            const auto t0 = clock::now();
            for(int i = 0; i < burst; ++i)
            {
                const shape& s = shapes[i % shapes.size()];
                rocm_sgemm_f32(0, 0, 0, dC, dA, dB, s.m, s.n, s.k, stream);
            }
            total += us_per(t0, clock::now(), burst);
            HIP_CHECK(hipStreamSynchronize(stream));
        }
        rocm_sgemm_config cfg;
        rocm_sgemm_find_config(shapes[0].m, shapes[0].n, shapes[0].k, 0, 0, 0, &cfg);
        std::printf("host_cost call  %-58s %8.3f us per call   (first shape: split_k %d)\n", what, total / rounds,
                    cfg.split_k);
    };
    call_cost("plain product (256^3)", {{256, 256, 256}});
    call_cost("plain product (1024^3)", {{1024, 1024, 1024}});
    call_cost("split-K product (1024 x 1024 x 16384)", {{1024, 1024, 16384}});
    call_cost("stream-K tail (2560^3)", {{2560, 2560, 2560}});
    call_cost("two planned shapes in turn", {{1536, 1200, 900}, {777, 2222, 1111}});
    call_cost("twenty planned shapes in turn", many);
    HIP_CHECK(hipFree(dA));
    HIP_CHECK(hipFree(dB));
    HIP_CHECK(hipFree(dC));
    HIP_CHECK(hipStreamDestroy(stream));
    return 0;
}

} // namespace

int main(int argc, char* argv[])
{
    options opt;
    for(int i = 1; i < argc; ++i)
    {
        const std::string arg = argv[i];
        if(arg == "--shapes" && i + 1 < argc)
            opt.shapes = parse_shapes(argv[++i]);
        else if(arg == "--batch_count" && i + 1 < argc)
            opt.batch_count = std::max(1, std::stoi(argv[++i]));
        else if(arg == "--warmup" && i + 1 < argc)
            opt.warmup = std::max(0, std::stoi(argv[++i]));
        else if(arg == "--iters" && i + 1 < argc)
            opt.iters = std::max(1, std::stoi(argv[++i]));
        else if(arg == "--identity_b")
            opt.identity_b = true;
        else if(arg == "--verify")
            opt.verify = true;
        else if(arg == "--vendor")
            opt.vendor = true;
        else if(arg == "--pmc")
            opt.pmc = true, opt.warmup = 2, opt.iters = 5, min_warm_ms = 0.0;
        else if(arg == "--counters")
            opt.counters = true;
        else if(arg == "--host_cost")
            opt.host_cost = true;
        else if(arg == "--mfma_ceiling")
            opt.mfma_ceiling = true;
        else if(arg == "--l2_to_lds")
            opt.l2_to_lds = true;
        else if(arg == "--uniform")
        {
            opt.uniform = true;
            if(i + 1 < argc && argv[i + 1][0] != '-') opt.seed = static_cast<unsigned>(std::stoul(argv[++i]));
        }
        else if(arg == "--cpu")
        {
            opt.cpu_threads = 0;
            if(i + 1 < argc && argv[i + 1][0] != '-') opt.cpu_threads = std::stoi(argv[++i]);
        }
        else if(arg == "--layouts" && i + 1 < argc)
        {
            std::stringstream ss(argv[++i]);
            std::string       tok;
            while(std::getline(ss, tok, ','))
            {
                if(tok.size() != 3 || tok.find_first_not_of("rc") != std::string::npos)
                {
                    std::cerr << "bad layout '" << tok << "': three letters r/c for A, B, C\n";
                    return 2;
                }
                opt.layouts.push_back(((tok[0] == 'c') << 2) | ((tok[1] == 'c') << 1) | (tok[2] == 'c'));
            }
        }
        else if(arg == "--help")
        {
            print_usage(argv[0]);
            return 0;
        }
        else if(arg.rfind("--benchmark_", 0) == 0)
        {
            // flags the reference forwards to Google Benchmark: accepted and ignored
        }
        else
        {
            std::cerr << "unknown argument '" << arg << "'\n";
            print_usage(argv[0]);
            return 2;
        }
    }
#ifndef BENCH_WITH_ROCBLAS
    if(opt.vendor)
    {
        std::cerr << "built without rocBLAS: --vendor is unavailable\n";
        return 2;
    }
#endif
    if(opt.host_cost)
    {
        return run_host_cost();
    }
    if(opt.mfma_ceiling)
    {
        return run_mfma_ceiling();
    }
    if(opt.l2_to_lds)
    {
        return run_l2_to_lds();
    }
    if(opt.counters)
    {
        // Counter collection starts other processes under rocprofv3 and must not hold the GPU
        // itself, so the timing table is produced by a child as well.
        std::string cmd = shell_quote(argv[0]);
        for(int i = 1; i < argc; ++i)
            if(std::string(argv[i]) != "--counters") cmd += " " + shell_quote(argv[i]);
        const int rc = std::system(cmd.c_str());
        if(rc != 0) return 1;
        return collect_counters(opt, argv[0]);
    }
    return run(opt);
}
