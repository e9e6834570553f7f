// Where the time of one GEMM launch goes, workgroup by workgroup.
//
// Built with ROCM_SGEMM_PHASE_STAMPS, which makes every wave of sgemm_mfma_kernel record the wall
// clock (100 MHz) at its start, after its prologue, after its main loop and after its last store
// has completed, the shader-clock cycles of its main loop and the XCD it ran on.  The library
// itself is built without the macro; this program instantiates the kernels it looks at and
// launches them directly, with the arguments the dispatcher would pass.
//
//   kernel_phases [case ...]        cases: 4096 8192 2048 1024 skinny ragged deepk   (default: all)
//
// For every case: warm-up of at least 100 ms, then launches queued back to back; the stamps are
// those of the last launch (the GPU is at its sustained clock).  Printed per XCD: mean start offset,
// prologue, main loop, epilogue (to the completion of the stores), end, and the shader clock in
// the main loop; then quantiles over the workgroups.  Times in microseconds.
// No counterpart in the reference (its bench reports one time per launch,
// benchmark/gemm/bench.cpp:107-135).

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "launch.hpp"

#ifndef ROCM_SGEMM_PHASE_STAMPS
#error "build with -DROCM_SGEMM_PHASE_STAMPS"
#endif

using namespace rocm_sgemm;

#define CHECK(expr)                                                                              \
    do                                                                                           \
    {                                                                                            \
        const hipError_t status_ = (expr);                                                       \
        if(status_ != hipSuccess)                                                                \
        {                                                                                        \
            std::fprintf(stderr, "HIP error %s at line %d\n", hipGetErrorString(status_), __LINE__); \
            return 1;                                                                            \
        }                                                                                        \
    } while(0)

// One plain product (or a K split whose partials are left in a workspace) with config Cfg on
// row-major A, B, C: X = A depth-contiguous, Y = B column-contiguous.
template<class Cfg>
int run_case(const char* title, int M, int N, int K, int group_m, int split)
{
    static_assert(Cfg::X_KC && !Cfg::Y_KC, "row-major A and B");
    const int  grid_m = (M + Cfg::BM - 1) / Cfg::BM, grid_n = (N + Cfg::BN - 1) / Cfg::BN;
    const int  k_tiles = (K + Cfg::BK - 1) / Cfg::BK;
    const bool full    = M % Cfg::BM == 0 && N % Cfg::BN == 0 && K % Cfg::BK == 0;
    if(full == Cfg::EDGE || k_tiles % split != 0)
    {
        std::fprintf(stderr, "%s: the case does not fit the kernel variant\n", title);
        return 1;
    }
    float *A, *B, *C, *partial = nullptr;
    CHECK(hipMalloc(&A, sizeof(float) * M * K));
    CHECK(hipMalloc(&B, sizeof(float) * K * N));
    CHECK(hipMalloc(&C, sizeof(float) * M * N));
    std::vector<float> h(static_cast<size_t>(std::max(M, N)) * K);
    for(size_t i = 0; i < h.size(); ++i)
        h[i] = static_cast<float>((i * 2654435761u >> 20) % 17) / 16.0f - 0.5f;
    CHECK(hipMemcpy(A, h.data(), sizeof(float) * M * K, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(B, h.data(), sizeof(float) * K * N, hipMemcpyHostToDevice));
    const unsigned      grid  = static_cast<unsigned>(grid_m) * grid_n * split;
    const int           waves = Cfg::NT / 64;
    unsigned long long* stamps;
    CHECK(hipMalloc(&stamps, sizeof(unsigned long long) * grid * waves * 8));

    kernel::gemm_args a;
    std::memset(&a, 0, sizeof(a));
    a.P = C, a.X = A, a.Y = B;
    a.rows = M, a.cols = N, a.depth = K;
    a.ldx = K, a.ldy = N, a.ldp = N;
    a.extent_x = static_cast<long long>(M) * K, a.extent_y = static_cast<long long>(K) * N;
    a.grid_m = grid_m, a.grid_n = grid_n, a.group_m = group_m;
    a.split_k = split, a.k_slice = (k_tiles / split) * Cfg::BK;
    a.tail_begin = grid_m * grid_n;
    a.stamps     = stamps;
    if(split > 1)
    {
        CHECK(hipMalloc(&partial, sizeof(float) * M * N * split));
        a.partial = partial;
    }

    const double flop = 2.0 * M * N * K;
    hipEvent_t   e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    float warmed = 0.0f;
    while(warmed < 100.0f)
    {
        CHECK(hipEventRecord(e0, nullptr));
        for(int i = 0; i < 8; ++i)
            CHECK(detail::launch_kernel<Cfg>(a, grid, 1, nullptr));
        CHECK(hipEventRecord(e1, nullptr));
        CHECK(hipEventSynchronize(e1));
        float ms = 0;
        CHECK(hipEventElapsedTime(&ms, e0, e1));
        warmed += ms;
    }
    const int launches = std::max(8, std::min(400, static_cast<int>(20.0e-3 / (flop / 150.0e12))));
    CHECK(hipEventRecord(e0, nullptr));
    for(int i = 0; i < launches; ++i)
        CHECK(detail::launch_kernel<Cfg>(a, grid, 1, nullptr));
    CHECK(hipEventRecord(e1, nullptr));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::vector<unsigned long long> st(static_cast<size_t>(grid) * waves * 8);
    CHECK(hipMemcpy(st.data(), stamps, st.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));

    unsigned long long first = ~0ull, last = 0;
    for(size_t w = 0; w < static_cast<size_t>(grid) * waves; ++w)
    {
        first = std::min(first, st[w * 8]);
        last  = std::max(last, st[w * 8 + 3]);
    }
    std::printf("\n%s: %d x %d x %d, %u workgroups of %d waves%s\n", title, M, N, K, grid, waves,
                split > 1 ? " (K split, partials left in the workspace)" : "");
    std::printf("  %d launches back to back: %.2f us each = %.1f TFLOP/s; last launch, first wave start to last store: %.2f us\n",
                launches, ms * 1e3 / launches, flop / (ms / launches) * 1e-9, (last - first) * 0.01);
    struct sums
    {
        double start = 0, prologue = 0, loop = 0, epilogue = 0, end = 0, mhz = 0, end_max = 0;
        int    n = 0;
    } xcd[8];
    std::vector<double> v_start, v_pro, v_loop, v_epi, v_end;
    double              skew_sum = 0, skew_max = 0;
    for(unsigned g = 0; g < grid; ++g)
    {
        const unsigned long long* o = &st[static_cast<size_t>(g) * waves * 8]; // wave 0 of the workgroup
        const double start = (o[0] - first) * 0.01, pro = (o[1] - o[0]) * 0.01, loop = (o[2] - o[1]) * 0.01;
        const double epi = (o[3] - o[2]) * 0.01, end = (o[3] - first) * 0.01;
        sums&        x   = xcd[o[5] & 7];
        x.start += start, x.prologue += pro, x.loop += loop, x.epilogue += epi, x.end += end;
        x.mhz += o[2] > o[1] ? static_cast<double>(o[4]) / static_cast<double>(o[2] - o[1]) * 100.0 : 0.0;
        x.end_max = std::max(x.end_max, end);
        ++x.n;
        v_start.push_back(start), v_pro.push_back(pro), v_loop.push_back(loop), v_epi.push_back(epi), v_end.push_back(end);
        double lo = 1e30, hi = 0;
        for(int w = 0; w < waves; ++w)
        {
            const double t = (st[(static_cast<size_t>(g) * waves + w) * 8 + 2] - first) * 0.01;
            lo = std::min(lo, t), hi = std::max(hi, t);
        }
        skew_sum += hi - lo, skew_max = std::max(skew_max, hi - lo);
    }
    std::printf("  XCD  workgroups   start  prologue      loop  epilogue       end   end max   shader clock in the loop\n");
    for(int i = 0; i < 8; ++i)
        if(xcd[i].n > 0)
        {
            const sums& x = xcd[i];
            std::printf("  %3d  %10d  %6.2f  %8.2f  %8.2f  %8.2f  %8.2f  %8.2f   %.0f MHz\n", i, x.n, x.start / x.n,
                        x.prologue / x.n, x.loop / x.n, x.epilogue / x.n, x.end / x.n, x.end_max, x.mhz / x.n);
        }
    const auto quantiles = [](std::vector<double> v, const char* what) {
        std::sort(v.begin(), v.end());
        const size_t n = v.size();
        std::printf("  %-9s min %8.2f  p10 %8.2f  p50 %8.2f  p90 %8.2f  max %8.2f\n", what, v[0], v[n / 10], v[n / 2],
                    v[n * 9 / 10], v[n - 1]);
    };
    quantiles(v_start, "start"), quantiles(v_pro, "prologue"), quantiles(v_loop, "loop");
    quantiles(v_epi, "epilogue"), quantiles(v_end, "end");
    std::printf("  end of the main loop, spread over the waves of a workgroup: mean %.2f, max %.2f\n", skew_sum / grid, skew_max);
    // MFMA cycles of one wave's main loop against the cycles it spent there, and - because waves that
    // share a SIMD take turns at its matrix pipe in no fixed pattern (a loop without stalls lets the
    // older wave run ahead and the younger one wait) - the share of all matrix-pipe cycles of the GPU
    // that MFMAs fill between the first wave entering its main loop and the last one leaving it.
    const double mfma_cycles = static_cast<double>(Cfg::TM * Cfg::TN) * (Cfg::MI == 32 ? 64.0 : 32.0)
                               * (static_cast<double>(K) / split) / (Cfg::MI == 32 ? 2.0 : 4.0) / Cfg::WK;
    int          cus = 256;
    (void)hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, 0);
    double             loop_cycles = 0, mhz = 0;
    unsigned long long loop_first = ~0ull, loop_last = 0;
    for(size_t w = 0; w < static_cast<size_t>(grid) * waves; ++w)
    {
        const unsigned long long* o = &st[w * 8];
        loop_cycles += static_cast<double>(o[4]);
        loop_first = std::min(loop_first, o[1]);
        loop_last  = std::max(loop_last, o[2]);
        mhz += o[2] > o[1] ? static_cast<double>(o[4]) / static_cast<double>(o[2] - o[1]) * 100.0 : 0.0;
    }
    loop_cycles /= static_cast<double>(grid) * waves;
    mhz /= static_cast<double>(grid) * waves;
    const double span_us    = (loop_last - loop_first) * 0.01;
    const double pipe_total = 4.0 * cus * span_us * mhz; // matrix-pipe cycles of the GPU in that span
    std::printf("  main loop: %.0f shader cycles per wave on average, %.0f of them its own MFMAs; from the first wave "
                "entering its loop to the last leaving (%.2f us at %.0f MHz): pipe busy %.1f %% of the loop\n",
                loop_cycles, mfma_cycles, span_us, mhz,
                mfma_cycles * static_cast<double>(grid) * waves / pipe_total * 100.0);
    CHECK(hipFree(A));
    CHECK(hipFree(B));
    CHECK(hipFree(C));
    CHECK(hipFree(stamps));
    if(partial != nullptr) CHECK(hipFree(partial));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return 0;
}

int main(int argc, char** argv)
{
    using kernel::tile_config;
    std::vector<std::string> cases;
    for(int i = 1; i < argc; ++i)
        cases.emplace_back(argv[i]);
    if(cases.empty()) cases = {"4096", "8192", "2048", "1024", "skinny", "ragged", "deepk"};
    int rc = 0;
    for(const std::string& c : cases)
    {
        if(c == "4096")
            rc |= run_case<tile_config<256, 256, 32, 2, 2, 32, true, false, false, 2, 4, 4, 1>>(
                "256x256x32, 2x2 waves, 2 stages", 4096, 4096, 4096, 4, 1);
        else if(c == "8192")
            rc |= run_case<tile_config<256, 256, 32, 2, 2, 32, true, false, false, 2, 4, 4, 1>>(
                "256x256x32, 2x2 waves, 2 stages", 8192, 8192, 8192, 4, 1);
        else if(c == "2048")
            rc |= run_case<tile_config<128, 128, 64, 4, 2, 32, true, false, false, 2, 4, 4, 1>>(
                "128x128x64, 4x2 waves, 2 stages", 2048, 2048, 2048, 4, 1);
        else if(c == "1024")
            rc |= run_case<tile_config<64, 64, 32, 2, 2, 32, true, false, false, 2, 4, 4, 1>>(
                "64x64x32, 2x2 waves, 2 stages", 1024, 1024, 1024, 4, 1);
        else if(c == "skinny")
            rc |= run_case<tile_config<64, 32, 64, 1, 1, 32, true, false, false, 3, 4, 4, 4>>(
                "64x32x64, 4 waves along K, 3 stages", 128, 4096, 4096, 4, 1);
        else if(c == "ragged")
            rc |= run_case<tile_config<64, 64, 32, 2, 2, 32, true, false, true, 3, 1, 1, 1>>(
                "64x64x32, 2x2 waves, 3 stages, masked with 4-byte loads", 1000, 3000, 777, 4, 1);
        else if(c == "deepk")
            rc |= run_case<tile_config<64, 64, 128, 1, 1, 32, true, false, false, 2, 4, 4, 4>>(
                "64x64x128, 4 waves along K, 2 stages", 1024, 1024, 16384, 4, 1);
        else
        {
            std::fprintf(stderr, "unknown case %s (4096 8192 2048 1024 skinny ragged deepk)\n", c.c_str());
            return 2;
        }
    }
    return rc;
}
