// What one instruction costs when it is issued into a stream of back-to-back MFMAs.
//
// The SGEMM main loop is a stream of v_mfma_f32_32x32x2_f32 (64 cycles of matrix pipe each) with
// data movement in between; whatever delays the next MFMA is lost matrix-pipe time.  This program
// measures that delay per kind of instruction: 256 workgroups of four waves (one per SIMD), 16
// independent accumulator tiles, 64 MFMAs per loop trip, one extra instruction every N MFMAs, and
// the shader-clock cycles of the loop per wave (s_memtime around it).
//
//   issue_cost
//
// Printed per kind: cycles per MFMA and the cycles one inserted instruction adds.  On MI355X:
// scalar-ALU instructions, LDS reads, direct-to-LDS loads (with their s_mov m0) and barriers add
// nothing measurable; one vector-ALU instruction adds about 13 cycles, a second one directly behind
// it about 4 more.  That is why the kernel's steady-state loop holds no vector-ALU instruction
// (csrc/sgemm_mfma_kernel.hpp: NS K-tiles per trip, constant stage indices).
// No counterpart in the reference, whose kernel has no matrix instructions
// (rocm_sgemm/include/rocm_sgemm/kernel/kernel.hpp:248-266 is a VALU FMA loop).

#include <algorithm>
#include <cstdio>
#include <type_traits>
#include <vector>

#include <hip/hip_runtime.h>

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __attribute__((address_space(3))) void lds_void;

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

template<int I, int N, class F>
__device__ __forceinline__ void static_for(F&& body)
{
    if constexpr(I < N)
    {
        body(std::integral_constant<int, I>{});
        static_for<I + 1, N>(body);
    }
}

enum kind
{
    NOTHING,
    VALU_ADD, // one v_add_u32 on registers nothing else uses
    VALU_ADD_TWICE, // two of them back to back
    SALU_ADDS, // four s_add_i32
    LDS_READ, // ds_read_b128 whose result feeds MFMAs of the next trip
    DMA_LOAD, // s_mov m0 + buffer_load_dwordx4 ... lds
    DMA_LOAD_DWORD, // s_mov m0 + buffer_load_dword ... lds
    BARRIER // s_barrier
};

// One extra instruction of kind KIND every EVERY MFMAs; 64 MFMAs per trip.
template<int KIND, int EVERY>
__global__ __launch_bounds__(256) void issue_cost_kernel(float* out, unsigned long long* cycles, const float* src,
                                                        int trips, int zero)
{
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int tid = threadIdx.x, lane = tid % 64, wave = __builtin_amdgcn_readfirstlane(tid / 64);
    for(int i = tid; i < 16384; i += 256)
        lds[i] = 0.001f * static_cast<float>(i % 97);
    __syncthreads();
    f32x16 acc[16];
    for(int t = 0; t < 16; ++t)
        for(int v = 0; v < 16; ++v)
            acc[t][v] = 0.0f;
    float fa[2][16], fb[16];
    for(int i = 0; i < 16; ++i)
        fa[0][i] = fa[1][i] = 1.0f + lane * 0.001f + i, fb[i] = 0.5f + i;
    int                          vx = lane, vy = zero, sx = zero;
    const float*                 window = lds + lane * 4 + wave * 1024;
    const __amdgpu_buffer_rsrc_t rsrc
        = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(src), 0, 1 << 20, 0x00020000);
    const unsigned long long c0 = clock64();
    for(int trip = 0; trip < trips; ++trip)
    {
        static_for<0, 2>([&](auto s_c) {
            constexpr int s = decltype(s_c)::value; // fragment set the MFMAs of this half read
            static_for<0, 32>([&](auto m_c) {
                constexpr int m = decltype(m_c)::value;
                if constexpr(m % EVERY == 0)
                {
                    constexpr int e = m / EVERY;
                    if constexpr(KIND == VALU_ADD) asm volatile("v_add_u32 %0, %0, %1" : "+v"(vx) : "v"(vy));
                    if constexpr(KIND == VALU_ADD_TWICE)
                        asm volatile("v_add_u32 %0, %0, %1\n\tv_add_u32 %0, %0, %1" : "+v"(vx) : "v"(vy));
                    if constexpr(KIND == SALU_ADDS)
                        asm volatile("s_add_i32 %0, %0, 1\n\ts_add_i32 %0, %0, 1\n\ts_add_i32 %0, %0, 1\n\ts_add_i32 %0, %0, 1"
                                     : "+s"(sx));
                    if constexpr(KIND == LDS_READ)
                    {
                        const f32x4 v    = *reinterpret_cast<const f32x4*>(window + (e % 4) * 256 + s * 4096);
                        constexpr int d  = (e * 4) % 16;
                        fa[s ^ 1][d]     = v.x;
                        fa[s ^ 1][d + 1] = v.y;
                        fa[s ^ 1][d + 2] = v.z;
                        fa[s ^ 1][d + 3] = v.w;
                    }
                    if constexpr(KIND == DMA_LOAD)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)(lds + 8192 + wave * 256 + (e % 8) * 1024),
                                                                 16, lane * 16, 0, 0, 0);
                    if constexpr(KIND == DMA_LOAD_DWORD)
                        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)(lds + 8192 + wave * 64 + (e % 8) * 256), 4,
                                                                 lane * 4, 0, 0, 0);
                    if constexpr(KIND == BARRIER) __builtin_amdgcn_s_barrier();
                }
                acc[m % 16] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s][(m / 4) % 16], fb[m % 16], acc[m % 16], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
        if constexpr(KIND == DMA_LOAD || KIND == DMA_LOAD_DWORD)
            __builtin_amdgcn_s_waitcnt(0x0F70); // vmcnt(0) once per trip
    }
    const unsigned long long c1  = clock64();
    float                    sum = static_cast<float>(vx + sx) + lds[8192 + tid];
    for(int t = 0; t < 16; ++t)
        for(int v = 0; v < 16; ++v)
            sum += acc[t][v];
    out[blockIdx.x * 256 + tid] = sum;
    if(lane == 0) cycles[blockIdx.x * 4 + tid / 64] = c1 - c0;
}

template<int KIND, int EVERY>
int run(const char* name, const float* src, double* per_mfma_out)
{
    const int           grid = 256, trips = 500;
    float*              out;
    unsigned long long* cyc;
    CHECK(hipMalloc(&out, grid * 256 * sizeof(float)));
    CHECK(hipMalloc(&cyc, grid * 4 * sizeof(unsigned long long)));
    CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(issue_cost_kernel<KIND, EVERY>),
                              hipFuncAttributeMaxDynamicSharedMemorySize, 65536));
    for(int w = 0; w < 30; ++w) // the last launch is the one read back: the GPU is at its sustained clock
        hipLaunchKernelGGL((issue_cost_kernel<KIND, EVERY>), dim3(grid), dim3(256), 65536, nullptr, out, cyc, src, trips, 0);
    CHECK(hipDeviceSynchronize());
    std::vector<unsigned long long> h(grid * 4);
    CHECK(hipMemcpy(h.data(), cyc, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
    double mean = 0;
    for(unsigned long long c : h)
        mean += static_cast<double>(c);
    mean /= static_cast<double>(h.size());
    const double per = mean / (trips * 64.0);
    if(per_mfma_out != nullptr) *per_mfma_out = per;
    std::printf("%-58s every %2d MFMAs: %7.3f cycles per MFMA\n", name, EVERY, per);
    CHECK(hipFree(out));
    CHECK(hipFree(cyc));
    return 0;
}

int main()
{
    float* src;
    CHECK(hipMalloc(&src, 1 << 20));
    CHECK(hipMemset(src, 0, 1 << 20));
    double base = 0, v = 0;
    int    rc   = run<NOTHING, 64>("nothing but MFMAs", src, &base);
    struct row
    {
        const char* name;
        double      per_mfma;
        int         every;
    };
    std::vector<row> rows;
    auto add = [&](const char* name, int every, double per) { rows.push_back(row{name, per, every}); };
    rc |= run<VALU_ADD, 8>("one vector-ALU add", src, &v), add("vector-ALU add", 8, v);
    rc |= run<VALU_ADD, 1>("one vector-ALU add", src, &v), add("vector-ALU add", 1, v);
    rc |= run<VALU_ADD_TWICE, 8>("two vector-ALU adds back to back", src, &v), add("two vector-ALU adds", 8, v);
    rc |= run<SALU_ADDS, 1>("four scalar-ALU adds", src, &v), add("four scalar-ALU adds", 1, v);
    rc |= run<LDS_READ, 8>("one ds_read_b128 (result used)", src, &v), add("ds_read_b128", 8, v);
    rc |= run<LDS_READ, 2>("one ds_read_b128 (result used)", src, &v), add("ds_read_b128", 2, v);
    rc |= run<DMA_LOAD, 4>("s_mov m0 + buffer_load_dwordx4 ... lds", src, &v), add("direct-to-LDS load, 16 bytes per lane", 4, v);
    rc |= run<DMA_LOAD_DWORD, 1>("s_mov m0 + buffer_load_dword ... lds", src, &v), add("direct-to-LDS load, 4 bytes per lane", 1, v);
    rc |= run<BARRIER, 16>("s_barrier", src, &v), add("s_barrier", 16, v);
    std::printf("\ncycles one inserted instruction (group) adds to the MFMA stream (MFMAs alone: %.3f cycles each)\n", base);
    for(const row& r : rows)
        std::printf("cost %-42s every %2d MFMAs: %6.2f cycles\n", r.name, r.every, (r.per_mfma - base) * r.every);
    CHECK(hipFree(src));
    return rc;
}
