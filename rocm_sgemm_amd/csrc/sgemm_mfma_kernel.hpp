// gfx950 (CDNA4, wave64) FP32 SGEMM kernel built on v_mfma_f32_32x32x2_f32 / v_mfma_f32_16x16x4_f32.
//
// This is the device side of rocm_sgemm::gemm; it takes the place of the reference's VALU kernel
// (rocm_sgemm/include/rocm_sgemm/kernel/kernel.hpp:66-362 and kernel/load.hpp:32-173) and is a new
// design, not a translation: plain IEEE fp32 multiply-add on the matrix cores, no reduced
// precision anywhere.
//
// The kernel always produces a ROW-MAJOR output P (rows x cols) = X (rows x depth) * Y (depth x cols).
// A column-major C is served by the host through C^T = B^T * A^T, i.e. by swapping the operands,
// so only the storage order of the two inputs is a template parameter:
//   X_KC = true  : X is stored depth-contiguous   (row-major   X, "k-contiguous")
//   X_KC = false : X is stored row-contiguous     (column-major X, "m-contiguous")
//   Y_KC = true  : Y is stored depth-contiguous   (column-major Y)
//   Y_KC = false : Y is stored column-contiguous  (row-major   Y)
//
// Data path per workgroup (macro tile BM x BN, K-tile BK, WM x WN waves), two variants:
//   direct-to-LDS (NS >= 2 stages; operands whose lines are 16-byte aligned):
//     HBM --buffer_load_dwordx4 ... lds, 128 bits per lane along the operand's contiguous
//          dimension, NS - 1 K-tiles ahead--> LDS ring of NS stages
//         --128-bit ds_read--> MFMA operand registers (one k-block ahead)
//     No register staging and no ds_write: next to back-to-back MFMAs an LDS store of staged
//     registers costs about 2 % of matrix-pipe time on this part, the DMA path does not.
//     With EDGE the loads are range-checked against the operand's end (rows beyond a depth-
//     contiguous operand and depth lines beyond a row-contiguous one arrive as zeros), the
//     16-byte pieces of a depth-contiguous row at or beyond K are rejected lane by lane (they
//     arrive as zeros too) and the stores are predicated, which covers ragged M, N and K as long
//     as the rows of a depth-contiguous operand end on a 16-byte boundary (K a multiple of 4).
//     With DGX == 1 (DGY == 1) the same kernel moves X (Y) 4 bytes per lane (buffer_load_dword
//     ... lds) into the same LDS image, which lifts every alignment requirement on that operand:
//     odd leading dimension, unaligned pointer, any K.  The granularity is a template parameter
//     per operand, but only the 16 / 16 and the 4 / 4 kernels are compiled: one misaligned operand
//     moves both to 4-byte loads (a 16 / 4 kernel measured 1 % faster where it applies).
//   register-staged (NS == 0; the alternative for shapes without an LDS ring):
//     HBM --128-bit buffer loads--> registers (one K-tile ahead)
//         --128-bit ds_write, same orientation as in memory--> LDS (two stages)
//         --128-bit ds_read--> MFMA operand registers (one k-block ahead)
// The LDS image keeps the orientation the operand has in HBM; the "transpose" the MFMA operand
// layout needs is done by choosing which four values one 128-bit LDS read delivers:
//   depth-contiguous image [row][k] : one read = 4 consecutive k of ONE row  -> feeds 4 MFMA k-steps
//   row-contiguous image   [k][row] : one read = 4 consecutive rows of ONE k -> feeds 4 MFMA tiles
// Waves along K (WK > 1): the WM x WN wave grid is replicated WK times and replica w multiplies
// only the k-blocks [w * NKB / WK, (w + 1) * NKB / WK) of every K-tile, over the whole wave tile;
// the WK partial tiles are summed through LDS before the store.  A 64 x 64 macro tile with WK = 4
// gives every wave a 64 x 64 wave tile (four independent accumulator tiles, one LDS read per four
// MFMAs) where the plain 2 x 2 wave grid gives it one 32 x 32 tile (a chain of dependent MFMAs and
// one read per two): small macro tiles, which small and skinny problems need to fill 256 CUs,
// then run the inner loop of a large one.
// An MI x MI MFMA (MI = 32: 32x32x2, MI = 16: 16x16x4) takes its row/column from lane % MI and its
// k from the lane group h = lane / MI (2 or 4 groups).  Inside every "k-block" of 4 * (64 / MI)
// k values (8 or 16), MFMA step r (0..3) multiplies k = 4*h + r; X and Y use the same assignment,
// and any consistent assignment gives the same dot products.  With a row-contiguous image the four
// tiles a lane feeds are interleaved (row = 4*lane + tile) instead of stacked, which also makes
// the output stores of a lane contiguous (128-bit) when Y is column-contiguous.
#ifndef ROCM_SGEMM_AMD_SGEMM_MFMA_KERNEL_HPP
#define ROCM_SGEMM_AMD_SGEMM_MFMA_KERNEL_HPP

#include <type_traits>

#include <hip/hip_runtime.h>

#include "tile_order.hpp"

namespace rocm_sgemm
{
namespace kernel
{

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
// Same vectors with element alignment only: rows of an operand whose leading dimension is not a
// multiple of four start at arbitrary 4-byte offsets.
typedef float f32x2_e __attribute__((ext_vector_type(2), aligned(4)));
typedef float f32x4_e __attribute__((ext_vector_type(4), aligned(4)));

/// Kernel arguments.  For every batch b = blockIdx.y:
///   P_b = X_b * Y_b,   P_b row-major rows x cols with row stride ldp,   Z_b = Z + b * stride_z.
struct gemm_args
{
    float*       P;
    const float* X;
    const float* Y;
    int          rows; // M of the (possibly swapped) problem
    int          cols; // N
    int          depth; // K
    // Leading dimensions in floats: distance between consecutive lines of the operand's
    // contiguous dimension (ldx: between rows of a depth-contiguous X, between depth lines of a
    // row-contiguous X; same for ldy with columns; ldp: between rows of P).
    int       ldx, ldy, ldp;
    long long stride_x, stride_y, stride_p; // batch strides in floats
    long long extent_x, extent_y; // floats from an operand's origin to one past its last element
    int          grid_m; // number of macro-tile rows
    int          grid_n; // number of macro-tile columns
    int          group_m; // tile-order band height
    int          split_k; // number of K slices (1 = none)
    int          k_slice; // depth per slice, multiple of BK (== depth when split_k == 1)
    float*       partial; // split_k > 1: workspace of split_k packed row-major rows x cols partials
                          // per batch; tail_groups > 0: 2 * tail_groups partial tiles, each BM x BN
    // Stream-K tail (only with split_k == 1 and one batch): the tiles whose sequence number is
    // >= tail_begin (a short last wave) are not given one workgroup each.  Their K-tiles, laid end
    // to end (tile-major), are dealt out in runs of tail_per K-tiles to tail_groups workgroups, so
    // that every CU works for the same time.  tail_per <= K-tiles per tile, hence a run touches at
    // most two tiles ("segments"); workgroup g stores the partial tile of its segment s at
    // partial[(2 g + s) * BM * BN] and tail_reduce_kernel sums the segments of every tile.
    int tail_begin; // == grid_m * grid_n when there is no tail
    int tail_groups; // 0 = none
    int tail_per;
    // Partial tiles summed inside this launch (split_k > 1 or a stream-K tail): one counter per
    // (batch, tile, wave of the workgroup), all zero when the launch starts and zero again when it
    // ends; the wave that completes a counter adds up the tile's parts and stores the result.
    // Null: the partial tiles are left for a second kernel.
    unsigned* counters;
#if defined(ROCM_SGEMM_PHASE_STAMPS)
    // Only in the build of benchmark/kernel_phases (never in the library): eight 64-bit words per
    // wave of the launch - wall clock (100 MHz) at the start of the kernel, after the prologue,
    // after the main loop of the last segment and after the last store has completed; shader-clock
    // cycles spent in that main loop; the XCD the wave ran on.
    unsigned long long* stamps;
#endif
};

template<int BM_, int BN_, int BK_, int WM_, int WN_, int MI_, bool X_KC_, bool Y_KC_, bool EDGE_, int NS_ = 0,
         int DGX_ = 4, int DGY_ = 4, int WK_ = 1>
struct tile_config
{
    static constexpr int  BM   = BM_;
    static constexpr int  BN   = BN_;
    static constexpr int  BK   = BK_;
    static constexpr int  WM   = WM_;
    static constexpr int  WN   = WN_;
    static constexpr int  MI   = MI_; // MFMA tile: 32 -> v_mfma_f32_32x32x2_f32, 16 -> v_mfma_f32_16x16x4_f32
    static constexpr bool X_KC = X_KC_;
    static constexpr bool Y_KC = Y_KC_;
    static constexpr bool EDGE = EDGE_;
    static constexpr int  NS   = NS_; // 0: register-staged, two LDS stages; >= 2: direct-to-LDS ring
    static constexpr bool DTL  = NS_ >= 2;
    // Direct-to-LDS granularity: floats each lane moves per load.  4 (buffer_load_dwordx4 ... lds)
    // needs 16-byte aligned global addresses; 1 (buffer_load_dword ... lds) needs none beyond the
    // element's own and serves operands whose lines start anywhere (odd leading dimensions,
    // unaligned pointers, any K), at four times the number of load instructions.
    static constexpr int DGX = DGX_; // X operand
    static constexpr int DGY = DGY_; // Y operand
    // Waves along K: the wave grid is replicated WK times, replica w works on the w-th part of the
    // k-blocks of every K-tile, and the partial tiles are summed through LDS at the end.
    static constexpr int WK = WK_;

    static constexpr int NT  = 64 * WM * WN * WK; // threads per workgroup
    static constexpr int WTM = BM / WM; // wave tile
    static constexpr int WTN = BN / WN;
    static constexpr int TM  = WTM / MI; // MFMA tiles per wave
    static constexpr int TN  = WTN / MI;
    static constexpr int ACC = MI * MI / 64; // accumulator registers per MFMA tile
    static constexpr int KB  = 4 * (64 / MI); // depth of a k-block: 4 MFMA steps
    static constexpr int NKB = BK / KB; // k-blocks per K-tile
    static constexpr int NKBW = NKB / WK; // k-blocks of a K-tile one wave multiplies
    // Whether the kernel can add up the partial tiles of a K split or a stream-K tail itself
    // (gemm_args::counters): a wave's share of the macro tile is at most 64 x 64, and the workgroup
    // has at most four waves (with eight, two waves share a SIMD's registers and the summing code
    // does not fit beside the accumulators).
    static constexpr bool SUMS_IN_LAUNCH = BM * BN / (WM * WN * WK) <= 64 * 64 && WM * WN * WK <= 4;

    // Interleave width of a row-contiguous operand (tiles fed by one LDS read).
    static constexpr int VM = TM >= 4 ? 4 : TM;
    static constexpr int VN = TN >= 4 ? 4 : TN;

    // LDS images, register-staged path.  Depth-contiguous: [row][BK + 4]; the +4 makes consecutive
    // rows start 4 banks apart (odd multiple of 4 because BK % 8 == 0), so a 128-bit read of 16
    // consecutive rows touches all 64 banks once.  Row-contiguous: [k][rows + 4]; reads are
    // contiguous across lanes.
    // Direct-to-LDS path: the hardware writes the 64 lanes of a load contiguously, so the images
    // are unpadded, [row][BK] and [k][rows]; a depth-contiguous image is kept conflict-free by
    // XOR-swizzling the 16-byte chunks of a row instead (impl::dma_map).
    static constexpr int PAD    = DTL ? 0 : 4;
    static constexpr int LDX    = X_KC ? BK + PAD : BM + PAD;
    static constexpr int LDY    = Y_KC ? BK + PAD : BN + PAD;
    static constexpr int X_SIZE = X_KC ? BM * LDX : BK * LDX;
    static constexpr int Y_SIZE = Y_KC ? BN * LDY : BK * LDY;
    static constexpr int STAGE  = X_SIZE + Y_SIZE;
    static constexpr int STAGES = DTL ? NS : 2;
    // WK > 1: after the main loop every wave-grid replica leaves its partial tile in LDS as an
    // unpadded BM x BN row-major image, which the workgroup then reads linearly (thread t the
    // t-th group of four floats: conflict-free).  The two lane groups of an MFMA tile write rows
    // that differ in bit EX_ROW_BIT and would hit the same banks; so bit 5 of an element's linear
    // index (32 floats = half of the 64 banks) is flipped where that row bit is set.
    static constexpr int EX_ROW_BIT = X_KC ? 2 : (VM == 4 ? 4 : (VM == 2 ? 3 : 2));
    static constexpr int EX_FLOATS  = WK > 1 ? WK * BM * BN : 0;
    static constexpr int LDS_FLOATS = STAGES * STAGE > EX_FLOATS ? STAGES * STAGE : EX_FLOATS;
    static constexpr int LDS_BYTES = LDS_FLOATS * 4;
    // Waves per SIMD the register allocator is held to.  Left to itself it sizes a kernel for one
    // workgroup per CU; a K-split kernel whose LDS lets two workgroups share a CU (128 x 64 and
    // 64 x 128 with WK = 2) then takes 264 - 270 registers for the summing code of the epilogue,
    // just over the 256 that two waves per SIMD leave each, and loses 5 % (2048^3: 131.6 against
    // 137.8 TFLOP/s).  The same goes for the other kernels whose waves hold 64 accumulator
    // registers (128 x 128 on 2 x 2 waves: the masked variants take 260 - 264 registers unbounded).
    static constexpr int WG_PER_CU_BY_LDS = 160 * 1024 / LDS_BYTES;
    static constexpr int MIN_WAVES_PER_SIMD
        = WG_PER_CU_BY_LDS >= 2 && ((WK > 1 && BM * BN / (WM * WN) >= 64 * 64) || BM * BN / (WM * WN * WK) == 64 * 64)
              ? 2 * ((NT / 64 + 3) / 4)
              : 1;

    // Swizzle of a depth-contiguous direct-to-LDS image: rows of BK floats, CPR 16-byte chunks
    // each, RPL rows per 64-bank line.
    static constexpr int CPR = BK / 4;
    static constexpr int RPL = 64 / BK > 0 ? 64 / BK : 1;

    // Pieces each thread moves per K-tile: 128-bit chunks, or DGX / DGY floats on the direct-to-LDS path.
    static constexpr int CX = BM * BK / (DTL ? DGX : 4) / NT;
    static constexpr int CY = BN * BK / (DTL ? DGY : 4) / NT;

    static_assert(MI == 32 || MI == 16, "MFMA tile is 32x32x2 or 16x16x4");
    static_assert(BM % (MI * WM) == 0 && BN % (MI * WN) == 0, "wave tile must be a multiple of the MFMA tile");
    static_assert(WK >= 1 && NKB % WK == 0 && (NKB / WK) % 2 == 0,
                  "every wave multiplies an even number of k-blocks of a K-tile");
    static_assert(WK == 1 || DTL, "waves along K exist for the direct-to-LDS kernels only");
    static_assert((BM * BN / 4) % NT == 0, "the summed tile must divide evenly among the threads");
    static_assert((DGX == 4 || DGX == 1) && (DGY == 4 || DGY == 1), "16-byte or 4-byte pieces");
    static_assert((DGX == 4 && DGY == 4) || (DTL && EDGE), "single-float loads exist for the masked direct-to-LDS kernel only");
    static_assert((BM * BK / 4) % NT == 0 && (BN * BK / 4) % NT == 0, "chunks must divide evenly");
    static_assert(TM == 1 || TM == 2 || TM % 4 == 0, "TM in {1,2,4,8,...}");
    static_assert(TN == 1 || TN == 2 || TN % 4 == 0, "TN in {1,2,4,8,...}");
    static_assert(LDS_BYTES <= 160 * 1024, "exceeds CDNA4 LDS");
    static_assert(NS == 0 || (NS >= 2 && NS <= 8), "0 (register-staged) or 2..8 LDS stages");
    static_assert(!DTL || (MI / RPL) % CPR == 0, "swizzle must not depend on the MFMA tile index");
};

namespace impl
{

constexpr int max_int(int a, int b)
{
    return a > b ? a : b;
}

// Number of items, out of n spread evenly over `span` slots (item e in slot e * span / n), that sit
// in slots before `slot`.
constexpr int items_before(int slot, int span, int n)
{
    return slot <= 0 ? 0 : (slot >= span ? n : (slot * n + span - 1) / span);
}

// Compile-time loop: body(std::integral_constant<int, I>) for I in [0, N).  The pipeline below is
// written with it so that every register-array index is a constant by construction rather than by
// the grace of the loop unroller.
template<int I, int N, class F>
__device__ __forceinline__ void static_for(F&& body)
{
    if constexpr(I < N)
    {
        body(std::integral_constant<int, I>{});
        static_for<I + 1, N>(body);
    }
}

// ---- global -> register staging ------------------------------------------------------------
//
// Loads go through buffer instructions: a wave-uniform base (the start of the operand's current
// K-tile, in a scalar buffer descriptor), a wave-uniform chunk offset in an SGPR and one
// thread-fixed 32-bit offset in a VGPR.  Compared with 64-bit per-lane global addresses this
// needs no address arithmetic in the loop and issues measurably faster next to MFMAs.

typedef int i32x4 __attribute__((ext_vector_type(4)));

// 128 bits at base + (voff + soff) floats; base, bytes and soff must be wave-uniform.  `bytes` is
// the size of the buffer starting at base: the hardware checks every dword of the access against
// it and returns 0.0f for those at or beyond the end (4-byte alignment is enough).
__device__ __forceinline__ f32x4 buffer_load_f32x4(const float* base, unsigned bytes, int voff, int soff)
{
#if defined(__HIP_DEVICE_COMPILE__)
    // raw buffer (stride 0); word 3 = 32-bit data format for gfx9-family descriptors
    const __amdgpu_buffer_rsrc_t rsrc
        = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, static_cast<int>(bytes), 0x00020000);
    const i32x4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff * 4, soff * 4, 0);
    return __builtin_bit_cast(f32x4, v);
#else
    (void)base, (void)bytes, (void)voff, (void)soff;
    return f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#endif
}

// Where chunk i of thread tid sits inside a K-tile.  Chunk q = i * NT + tid covers
//   KC: row q / (BK/4), k (q % (BK/4)) * 4        (ld = depth of the full matrix)
//   RC: k   q / (R/4),  row (q % (R/4)) * 4       (ld = rows of the full matrix)
// Because NT is a multiple of the chunks per line, the position splits into a part that depends
// only on the thread and a part that depends only on i.
template<bool KC, int R, int BK, int NT>
struct chunk_map
{
    static constexpr int LINE = KC ? BK / 4 : R / 4; // chunks per contiguous line
    static constexpr int STEP = NT / LINE; // lines advanced per chunk index i
    static_assert(NT % LINE == 0, "threads must cover whole lines");

    // line = row (KC) or k (RC); pos = k (KC) or row (RC), both inside the tile
    __device__ __forceinline__ static int line(int i, int tid)
    {
        return i * STEP + tid / LINE;
    }
    __device__ __forceinline__ static int pos(int tid)
    {
        return (tid % LINE) * 4;
    }
    // float offsets from the tile origin: thread part and uniform part
    __device__ __forceinline__ static int thread_offset(int tid, int ld)
    {
        return (tid / LINE) * ld + pos(tid);
    }
    __device__ __forceinline__ static int chunk_offset(int i, int ld)
    {
        return i * STEP * ld;
    }
};

// Loads chunk i of the K-tile whose origin is `tile` (first row of the panel, first depth of the
// tile); `bytes` = size of the operand from that origin to its end.
//
// Edge handling is branch-free.  Everything past the END OF THE OPERAND reads as zero through the
// buffer range check: rows beyond the matrix of a depth-contiguous operand, and depth lines beyond
// K of a row-contiguous one.  What remains:
//   * depth-contiguous operand, ragged K: the tail of a row's last chunk lies in the next row, so
//     those elements are zeroed explicitly (4 selects);
//   * row-contiguous operand, rows beyond the matrix: they read the next depth line.  That data
//     only ever reaches accumulators of output rows (columns) beyond M (N), which are never
//     stored, so it is left alone.
template<bool KC, int R, int BK, int NT>
__device__ __forceinline__ f32x4 load_chunk(int i, const float* tile, unsigned bytes, int voff, int ld)
{
    using map = chunk_map<KC, R, BK, NT>;
    return buffer_load_f32x4(tile, bytes, voff, map::chunk_offset(i, ld));
}

// The explicit zeroing of a depth-contiguous chunk's tail past the depth range (see above).  It is
// applied when the staged register is consumed, not when it is loaded, so that it does not wait
// on the load.  `k_rem` = valid depth from the origin of the tile the chunk belongs to.
template<bool KC, bool EDGE, int R, int BK, int NT>
__device__ __forceinline__ f32x4 mask_chunk(f32x4 v, int k_rem, int tid)
{
    if constexpr(EDGE && KC)
    {
        const int valid = k_rem - chunk_map<KC, R, BK, NT>::pos(tid);
        v.x             = valid > 0 ? v.x : 0.0f;
        v.y             = valid > 1 ? v.y : 0.0f;
        v.z             = valid > 2 ? v.z : 0.0f;
        v.w             = valid > 3 ? v.w : 0.0f;
    }
    return v;
}

// ---- register staging -> LDS (same orientation as in memory) ----------------------------------

template<bool KC, int R, int BK, int LD, int NT>
__device__ __forceinline__ void store_chunk(int i, float* __restrict__ lds, const f32x4& value, int tid)
{
    const int q = i * NT + tid;
    if constexpr(KC)
    {
        const int r = q / (BK / 4);
        const int k = (q % (BK / 4)) * 4;
        *reinterpret_cast<f32x4*>(lds + r * LD + k) = value;
    }
    else
    {
        const int k = q / (R / 4);
        const int r = (q % (R / 4)) * 4;
        *reinterpret_cast<f32x4*>(lds + k * LD + r) = value;
    }
}

// ---- HBM -> LDS without registers (direct-to-LDS path) ---------------------------------------

#if defined(__HIP_DEVICE_COMPILE__)
typedef __attribute__((address_space(3))) void lds_void;
#endif

// One wave-level transfer of 64 x G floats: lane L reads 4 G bytes at base + (voff + soff) floats
// and the hardware writes them at lds_dst + 4 G L bytes (lds_dst is wave-uniform and goes
// through M0).  Completion is counted by vmcnt like any other load.  The global address must be
// aligned to the size of the lane's piece (16 bytes for G = 4, 4 for G = 1).
template<int G>
__device__ __forceinline__ void dma_load(const float* base, unsigned bytes, int voff, int soff, float* lds_dst)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const __amdgpu_buffer_rsrc_t rsrc
        = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, static_cast<int>(bytes), 0x00020000);
    static_assert(G == 4 || G == 1, "16-byte or 4-byte pieces");
    const int voff_bytes = static_cast<int>(static_cast<unsigned>(voff) * 4u);
    if constexpr(G == 4) // the size operand must be a literal
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)(lds_dst), 16, voff_bytes, soff * 4, 0, 0);
    else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void*)(lds_dst), 4, voff_bytes, soff * 4, 0, 0);
#else
    (void)base, (void)bytes, (void)voff, (void)soff, (void)lds_dst;
#endif
}

// Workgroup barrier of the direct-to-LDS pipeline: waits until at most N of this wave's loads are
// still in flight and all of its LDS reads have returned, then joins the barrier.  Once every wave
// is through, the K-tile whose loads were waited for is complete in LDS (a load's vmcnt drops
// when its data is written) and the stage whose reads were waited for may be overwritten.
// This is deliberately not __syncthreads(): its fence makes the compiler wait for ALL outstanding
// loads (vmcnt(0)), which would drain the ring at every K-tile and leave deeper rings pointless.
// (gfx9 s_waitcnt encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] at [15:14].)
template<int N>
__device__ __forceinline__ void ring_barrier()
{
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
    __builtin_amdgcn_s_barrier();
#endif
}

// s_waitcnt vmcnt(0) alone.
__device__ __forceinline__ void wait_all_loads()
{
#if defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_waitcnt((7 << 4) | (15 << 8));
#endif
}

// Placement of the direct-to-LDS path.  Each lane moves a piece of G floats (4: a 16-byte chunk,
// 1: a single float).  Piece q = i * NT + tid lands at LDS float offset G * q of its operand's
// image, because a wave's 64 lanes are written contiguously: the images are the plain [row][BK]
// (depth-contiguous) and [k][R] (row-contiguous) arrays.
// A [row][BK] image read by 16 consecutive rows at one chunk position would hit the same few
// banks, so the 16-byte chunks of a row are XOR-swizzled: slot (row, p) holds the row's logical
// chunk p ^ swz(row), swz(row) = (row / RPL) % CPR.  The swizzle is applied on the global side (the
// lanes that own slot p fetch chunk p ^ swz(row)); a 128-byte row segment is still fetched by
// adjacent lanes, so the loads stay coalesced.
template<bool KC, int R, int BK, int NT, int G = 4>
struct dma_map
{
    static constexpr int CPR  = BK / 4;
    static constexpr int RPL  = 64 / BK > 0 ? 64 / BK : 1;
    static constexpr int LINE = (KC ? BK : R) / G; // pieces per contiguous line
    static constexpr int STEP = NT / LINE; // lines advanced per piece index i
    static constexpr int PPC  = 4 / G; // pieces per 16-byte chunk
    static_assert(NT % LINE == 0, "threads must cover whole lines");
    static_assert(!KC || STEP % RPL == 0, "a step must not split a bank line's rows");
    // A thread's offset depends on i through the swizzle of its row only (besides the uniform
    // i * STEP * ld), and that repeats with this period in i; 1 = the same offset for every i.
    static constexpr int gcd(int a, int b)
    {
        return b == 0 ? a : gcd(b, a % b);
    }
    static constexpr int PERIOD = KC ? CPR / gcd(STEP / RPL, CPR) : 1;

    __device__ __forceinline__ static constexpr int swz(int row)
    {
        return (row / RPL) % CPR;
    }
    // depth-contiguous image: position along K, within the K-tile, of the first float of piece i
    __device__ __forceinline__ static int depth_pos(int i, int tid)
    {
        const int line = i * STEP + tid / LINE;
        const int slot = tid % LINE;
        return ((slot / PPC) ^ swz(line)) * 4 + (slot % PPC) * G;
    }
    // float offset of piece i of thread tid from the K-tile origin, without the uniform
    // i * STEP * ld (lines advanced by the piece index)
    __device__ __forceinline__ static int lane_offset(int i, int tid, int ld)
    {
        return (tid / LINE) * ld + (KC ? depth_pos(i, tid) : (tid % LINE) * G);
    }
};

// Per-lane offset (in floats) that the range check of an edge-masked direct-to-LDS load always
// rejects: 2 GiB, while those loads declare at most 2 GiB - 1 bytes of operand.  A rejected lane
// writes zeros to LDS.
constexpr int dma_reject = 0x20000000;
constexpr unsigned dma_max_bytes = 0x7FFFFFFFu;

// ---- LDS -> MFMA operand fragments ---------------------------------------------------------------

// frag[t][r] = operand value this lane feeds to MFMA tile t at k-step r of a k-block.  One k-block
// of one operand takes read_count() LDS reads; read_one() performs read number q of them:
//   depth-contiguous image: q = tile,            one 128-bit read = the 4 k-steps of that tile
//   row-contiguous image:   q = r * (T/V) + g,   one read of V floats = tiles g*V .. g*V+V-1 at step r
template<bool KC, int T, int V>
__device__ __forceinline__ constexpr int read_count()
{
    return KC ? T : 4 * (T / V);
}

//
// `swz_base` (SWZ: direct-to-LDS depth-contiguous image, otherwise unused): per-thread float offset, for
// every k-block, of the swizzled chunk this lane reads in row w0 + c; tile q adds MI * q rows.
template<bool KC, bool SWZ, int T, int V, int LD, int MI>
__device__ __forceinline__ void read_one(int q, float (&frag)[T][4], const float* __restrict__ lds,
                                         const int* swz_base, int w0, int kb, int h, int c)
{
    constexpr int KB = 4 * (64 / MI);
    if constexpr(KC)
    {
        const float* p = SWZ ? lds + swz_base[kb] + MI * q * LD
                             : lds + (w0 + MI * q + c) * LD + kb * KB + 4 * h;
        const f32x4  v = *reinterpret_cast<const f32x4*>(p);
        frag[q][0]    = v.x;
        frag[q][1]    = v.y;
        frag[q][2]    = v.z;
        frag[q][3]    = v.w;
    }
    else
    {
        const int    r = q / (T / V);
        const int    g = q % (T / V);
        const float* p = lds + (kb * KB + 4 * h + r) * LD + w0 + g * MI * V + V * c;
        if constexpr(V == 4)
        {
            const f32x4 v      = *reinterpret_cast<const f32x4*>(p);
            frag[g * 4 + 0][r] = v.x;
            frag[g * 4 + 1][r] = v.y;
            frag[g * 4 + 2][r] = v.z;
            frag[g * 4 + 3][r] = v.w;
        }
        else if constexpr(V == 2)
        {
            const f32x2 v      = *reinterpret_cast<const f32x2*>(p);
            frag[g * 2 + 0][r] = v.x;
            frag[g * 2 + 1][r] = v.y;
        }
        else
        {
            frag[g][r] = *p;
        }
    }
}

// Row (or column) inside the wave tile that MFMA tile t, MFMA index i (0..MI-1) refers to.
template<bool KC, int V, int MI>
__device__ __forceinline__ constexpr int tile_index(int t, int i)
{
    if constexpr(KC)
    {
        return MI * t + i;
    }
    else
    {
        return (t / V) * MI * V + V * i + t % V;
    }
}

// One MFMA step on an MI x MI accumulator tile.
template<int MI, class Acc>
__device__ __forceinline__ Acc mfma(float a, float b, Acc acc)
{
    if constexpr(MI == 32)
        return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, acc, 0, 0, 0);
}

// MFMA row of accumulator register v of a lane in group h (the column is lane % MI):
//   32x32: v in 0..15 -> 8*(v/4) + 4*h + v%4        16x16: v in 0..3 -> 4*h + v
template<int MI>
__device__ __forceinline__ constexpr int acc_row(int v, int h)
{
    return MI == 32 ? 8 * (v / 4) + 4 * h + v % 4 : 4 * h + v;
}

} // namespace impl

template<class Cfg>
__global__ __launch_bounds__(Cfg::NT, Cfg::MIN_WAVES_PER_SIMD) void sgemm_mfma_kernel(const gemm_args args)
{
    constexpr int  BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK;
    constexpr int  TM = Cfg::TM, TN = Cfg::TN, NT = Cfg::NT, NKB = Cfg::NKBW, WK = Cfg::WK;
    constexpr bool X_KC = Cfg::X_KC, Y_KC = Cfg::Y_KC, EDGE = Cfg::EDGE, DTL = Cfg::DTL;
    constexpr int  VM = Cfg::VM, VN = Cfg::VN, MI = Cfg::MI, ACC = Cfg::ACC;
    constexpr int  NS = Cfg::STAGES;
    typedef float acc_t __attribute__((ext_vector_type(ACC)));

    // The only LDS object of the kernel, on purpose: with a second __shared__ variable the compiler
    // can no longer tell which object a direct-to-LDS load writes and waits for all loads in flight
    // (s_waitcnt vmcnt(0)) before every ds_read, which empties the ring (4096^3: 899 -> 1022 us).
    __shared__ __attribute__((aligned(16))) float lds[Cfg::LDS_FLOATS];

    const int tid  = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid / 64);
    const int lane = tid % 64;
    const int h    = lane / MI; // lane group: selects k inside an MFMA
    const int c    = lane % MI; // row (X operand) / column (Y operand) inside an MFMA tile
    const int wk   = wave / (Cfg::WM * Cfg::WN); // replica of the wave grid = part of every K-tile
    const int wmn  = wave % (Cfg::WM * Cfg::WN);
    const int wm0  = (wmn / Cfg::WN) * Cfg::WTM;
    const int wn0  = (wmn % Cfg::WN) * Cfg::WTN;
    const int kb0  = wk * NKB; // first k-block of a K-tile this wave multiplies

    // Workgroup -> one or two segments (tile, K range).
    //   ids below tail_begin (all ids when there is no tail): one segment.  With split_k > 1 every
    //                    tile has split_k slices; the slice is the slow index of the sequence that
    //                    is dealt out to the XCDs in contiguous chunks.
    //   ids from tail_begin on: workgroup g of the stream-K tail owns K-tiles [g * tail_per,
    //                    (g + 1) * tail_per) of the tail tiles laid end to end, i.e. a piece of one
    //                    tile and possibly the beginning of the next.
    const int  tiles   = args.grid_m * args.grid_n;
    const int  k_tiles = (args.depth + BK - 1) / BK;
    const bool tail    = args.tail_groups > 0 && static_cast<int>(blockIdx.x) >= args.tail_begin;
    const int  tail_g  = static_cast<int>(blockIdx.x) - args.tail_begin;
    int        run0 = 0, run1 = 0, tail_u0 = 0, nseg = 1;
    if(tail)
    {
        run0    = tail_g * args.tail_per;
        run1    = min(run0 + args.tail_per, (tiles - args.tail_begin) * k_tiles);
        tail_u0 = run0 / k_tiles;
        nseg    = (run1 - 1) / k_tiles > tail_u0 ? 2 : 1;
    }

#if defined(ROCM_SGEMM_PHASE_STAMPS)
    const unsigned long long stamp_start = wall_clock64();
    unsigned long long       stamp_loop_begin = 0, stamp_loop_end = 0, stamp_cycles = 0;
#endif
    const int batch             = blockIdx.y;
    const float* __restrict__ X = args.X + batch * args.stride_x;
    const float* __restrict__ Y = args.Y + batch * args.stride_y;
    const int ldx               = args.ldx;
    const int ldy               = args.ldy;

    // State of the current segment (set at the top of the segment loop below).
    int          slice = 0, wg = 0, m0 = 0, n0 = 0, k_begin = 0, k_end = 0, ntiles = 0;
    const float* x_panel = nullptr; // first row of the segment's tile, depth 0
    const float* y_panel = nullptr;

    acc_t acc[TM][TN];

    constexpr int CX = Cfg::CX, CY = Cfg::CY;
    constexpr int NRX = impl::read_count<X_KC, TM, VM>();
    constexpr int NRY = impl::read_count<Y_KC, TN, VN>();

    auto x_tile = [&](int t) { // origin of K-tile t of the X panel
        const size_t k0 = static_cast<size_t>(k_begin + t * BK);
        return x_panel + (X_KC ? k0 : k0 * ldx);
    };
    auto y_tile = [&](int t) {
        const size_t k0 = static_cast<size_t>(k_begin + t * BK);
        return y_panel + (Y_KC ? k0 : k0 * ldy);
    };

    // ---- data movement of one K-tile, cut into single instructions ("items") so that the main
    // loop can hand them out one at a time between MFMAs -----------------------------------------

    // register-staged path: thread-fixed offsets, staging registers, range-checked loads
    using map_x              = impl::chunk_map<X_KC, BM, BK, NT>;
    using map_y              = impl::chunk_map<Y_KC, BN, BK, NT>;
    // Everything below that depends on the lane (offsets into the operands, LDS addresses) is set
    // up by lane_setup() at the start of every segment, from a copy of the thread index that the
    // compiler cannot see through: computed once ahead of the segment loop, those registers would
    // stay occupied through the epilogue, which needs every register it can get.
    int tid_s = tid, h_s = h, c_s = c;
    int x_voff = 0, y_voff = 0;
    const float* const x_end  = X + args.extent_x;
    const float* const y_end  = Y + args.extent_y;
    auto               bytes_to = [](const float* from, const float* end) -> unsigned {
        const long long n = (end - from) * 4ll;
        return n <= 0 ? 0u : (n >= 0xFFFFFFFFll ? 0xFFFFFFFFu : static_cast<unsigned>(n));
    };
    f32x4 stage_x[DTL ? 1 : CX];
    f32x4 stage_y[DTL ? 1 : CY];
    auto  load_item = [&](int i, int t) { // global -> staging register i, K-tile t
        if constexpr(!DTL)
        {
            if(i < CX)
            {
                const float* tile = x_tile(t);
                stage_x[i] = impl::load_chunk<X_KC, BM, BK, NT>(i, tile, bytes_to(tile, x_end), x_voff, ldx);
            }
            else
            {
                const float* tile = y_tile(t);
                stage_y[i - CX]
                    = impl::load_chunk<Y_KC, BN, BK, NT>(i - CX, tile, bytes_to(tile, y_end), y_voff, ldy);
            }
        }
    };
    // `ragged_c`: the K-tile may be the last one of a depth that is not a multiple of BK, so what lies
    // beyond K is masked; a std::false_type caller guarantees a whole K-tile and pays for no masks
    auto store_item = [&](int i, int buf, int t, auto ragged_c) { // staging register i (K-tile t) -> LDS stage buf
        if constexpr(!DTL)
        {
            constexpr bool masked = EDGE && decltype(ragged_c)::value;
            float*         sx     = lds + buf * Cfg::STAGE;
            const int      k_rem  = k_end - (k_begin + t * BK);
            if(i < CX)
                impl::store_chunk<X_KC, BM, BK, Cfg::LDX, NT>(
                    i, sx, impl::mask_chunk<X_KC, masked, BM, BK, NT>(stage_x[i], k_rem, tid_s), tid_s);
            else
                impl::store_chunk<Y_KC, BN, BK, Cfg::LDY, NT>(
                    i - CX, sx + Cfg::X_SIZE,
                    impl::mask_chunk<Y_KC, masked, BN, BK, NT>(stage_y[i - CX], k_rem, tid_s), tid_s);
        }
    };

    // direct-to-LDS path: every access of a full tile is inside the operand, so there the buffer
    // range is left wide open and costs no per-tile arithmetic; the edge-masked variant passes the
    // distance to the operand's end, beyond which the hardware delivers zeros
    constexpr int DGX = Cfg::DGX, DGY = Cfg::DGY;
    using dma_x = impl::dma_map<X_KC, BM, BK, NT, DGX>;
    using dma_y = impl::dma_map<Y_KC, BN, BK, NT, DGY>;
    // per-lane offsets: piece i uses entry i % PERIOD (plus the uniform i * STEP * ld)
    constexpr int NVX = !DTL ? 1 : (dma_x::PERIOD < CX ? dma_x::PERIOD : CX);
    constexpr int NVY = !DTL ? 1 : (dma_y::PERIOD < CY ? dma_y::PERIOD : CY);
    int           x_doff[NVX];
    int           y_doff[NVY];
    // edge-masked variant, depth-contiguous operand: where along K each of the lane's pieces starts.
    // A row of such an operand continues into the next row, not into zeros, so in a ragged last
    // K-tile the pieces at or beyond the end of K (whole pieces: K is a multiple of the piece
    // size here) are rejected lane by lane; rows beyond the operand and the depth lines of a
    // row-contiguous operand beyond K lie behind the operand's end and are rejected by the range
    // check itself.
    int x_dpos[DTL && EDGE && X_KC ? NVX : 1];
    int y_dpos[DTL && EDGE && Y_KC ? NVY : 1];
    auto dma_item = [&](int i, int t, int buf, auto ragged_c) { // HBM -> LDS stage buf, piece i of K-tile t
        if constexpr(DTL)
        {
            constexpr bool masked = EDGE && decltype(ragged_c)::value; // see store_item
            float*         st     = lds + buf * Cfg::STAGE;
            const int      k_rem  = k_end - (k_begin + t * BK); // depth left from this K-tile's origin
            if(i < CX)
            {
                int       voff = x_doff[i % NVX];
                const int soff = i * dma_x::STEP * ldx;
                if constexpr(masked && X_KC)
                    voff = x_dpos[i % NVX] < k_rem ? voff : impl::dma_reject;
                const float* tile = x_tile(t);
                impl::dma_load<DGX>(tile, EDGE ? min(bytes_to(tile, x_end), impl::dma_max_bytes) : 0x7FFFFFFFu,
                                    voff, soff, st + (i * NT + wave * 64) * DGX);
            }
            else
            {
                const int j    = i - CX;
                int       voff = y_doff[j % NVY];
                const int soff = j * dma_y::STEP * ldy;
                if constexpr(masked && Y_KC)
                    voff = y_dpos[j % NVY] < k_rem ? voff : impl::dma_reject;
                const float* tile = y_tile(t);
                impl::dma_load<DGY>(tile, EDGE ? min(bytes_to(tile, y_end), impl::dma_max_bytes) : 0x7FFFFFFFu,
                                    voff, soff, st + Cfg::X_SIZE + (j * NT + wave * 64) * DGY);
            }
        }
    };

    // LDS -> fragments.  For a swizzled depth-contiguous image the chunk a lane reads in k-block kb
    // is (kb * KBC + h) ^ swz(row) = (kb * KBC) ^ (h ^ swz(row)): one base offset per k-block.
    constexpr int KBC = 64 / MI; // 16-byte chunks of a row per k-block and lane group
    int           xs_base[DTL && X_KC ? NKB : 1];
    int           ys_base[DTL && Y_KC ? NKB : 1];
    auto lane_setup = [&]() {
#if defined(__HIP_DEVICE_COMPILE__)
        tid_s = tid;
        asm volatile("" : "+v"(tid_s));
#endif
        h_s = (tid_s % 64) / MI;
        c_s = (tid_s % 64) % MI;
        if constexpr(!DTL)
        {
            x_voff = map_x::thread_offset(tid_s, ldx);
            y_voff = map_y::thread_offset(tid_s, ldy);
        }
        else
        {
            impl::static_for<0, NVX>([&](auto i) { x_doff[decltype(i)::value] = dma_x::lane_offset(decltype(i)::value, tid_s, ldx); });
            impl::static_for<0, NVY>([&](auto i) { y_doff[decltype(i)::value] = dma_y::lane_offset(decltype(i)::value, tid_s, ldy); });
            if constexpr(EDGE && X_KC)
                impl::static_for<0, NVX>([&](auto i) { x_dpos[decltype(i)::value] = dma_x::depth_pos(decltype(i)::value, tid_s); });
            if constexpr(EDGE && Y_KC)
                impl::static_for<0, NVY>([&](auto i) { y_dpos[decltype(i)::value] = dma_y::depth_pos(decltype(i)::value, tid_s); });
        }
        if constexpr(DTL && X_KC)
        {
            const int u = h_s ^ dma_x::swz(c_s);
            impl::static_for<0, NKB>([&](auto kb) {
                xs_base[decltype(kb)::value] = (wm0 + c_s) * BK + ((((kb0 + decltype(kb)::value) * KBC) ^ u) * 4);
            });
        }
        if constexpr(DTL && Y_KC)
        {
            const int u = h_s ^ dma_y::swz(c_s);
            impl::static_for<0, NKB>([&](auto kb) {
                ys_base[decltype(kb)::value] = (wn0 + c_s) * BK + ((((kb0 + decltype(kb)::value) * KBC) ^ u) * 4);
            });
        }
    };
    float fx[2][TM][4];
    float fy[2][TN][4];
    // depth offset of this wave's k-blocks inside an image that is not addressed through the
    // swizzle table above: depth lines of a row-contiguous image, floats of an unswizzled row
    const int x_koff = (X_KC ? (DTL ? 0 : 1) : Cfg::LDX) * (kb0 * Cfg::KB);
    const int y_koff = (Y_KC ? (DTL ? 0 : 1) : Cfg::LDY) * (kb0 * Cfg::KB);
    auto  read_item = [&](int q, int slot, int buf, int kb) { // LDS stage buf -> fragment set slot
        const float* sx = lds + buf * Cfg::STAGE;
        if(q < NRX)
            impl::read_one<X_KC, DTL, TM, VM, Cfg::LDX, MI>(q, fx[slot], sx + x_koff, xs_base, wm0, kb, h_s, c_s);
        else
            impl::read_one<Y_KC, DTL, TN, VN, Cfg::LDY, MI>(q - NRX, fy[slot], sx + Cfg::X_SIZE + y_koff,
                                                            ys_base, wn0, kb, h_s, c_s);
    };

    for(int seg = 0; seg < nseg; ++seg)
    {
    lane_setup();
    if(tail)
    {
        const int u = tail_u0 + seg;
        wg          = args.tail_begin + u;
        k_begin     = (max(run0, u * k_tiles) - u * k_tiles) * BK;
        k_end       = min(args.depth, (min(run1, (u + 1) * k_tiles) - u * k_tiles) * BK);
    }
    else if(args.split_k > 1)
    {
        // K slices: the whole (slice, tile) sequence, slice-major, is cut into one contiguous chunk
        // per XCD, so an XCD works on the tiles of one slice (or of a few): its workgroups share
        // one K range of both operands in its L2 instead of the whole depth of a few panels
        const int seq = detail::xcd_chunked_index(blockIdx.x, tiles * args.split_k);
        slice         = seq / tiles;
        wg            = seq - slice * tiles;
        k_begin       = slice * args.k_slice;
        k_end         = min(args.depth, k_begin + args.k_slice);
    }
    else
    {
        wg      = blockIdx.x;
        k_begin = 0;
        k_end   = args.depth;
    }
    {
        const detail::tile_coord tc
            = !tail && args.split_k > 1
                  ? detail::banded_tile(wg, args.grid_m, args.grid_n, args.group_m < 1 ? 1 : args.group_m)
                  : detail::map_workgroup(wg, args.grid_m, args.grid_n, args.group_m);
        m0 = tc.tile_m * BM;
        n0 = tc.tile_n * BN;
    }
    ntiles  = (k_end - k_begin + BK - 1) / BK;
    x_panel = X + (X_KC ? static_cast<size_t>(m0) * ldx : static_cast<size_t>(m0));
    y_panel = Y + (Y_KC ? static_cast<size_t>(n0) * ldy : static_cast<size_t>(n0));
    // The accumulators start at zero: each tile is cleared by one MFMA of zeros onto the constant
    // 0 (0 * 0 + 0), which lands in the accumulation registers directly.  From a plain `= 0.0f`
    // the compiler sometimes builds a vector of zeros in ordinary registers, keeps it across the
    // segment loop and spills it.
    {
        float nothing = 0.0f;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(nothing)); // one register holding 0.0f, not a constant the compiler can see through
#endif
#pragma unroll
        for(int i = 0; i < TM; ++i)
#pragma unroll
            for(int j = 0; j < TN; ++j)
                acc[i][j] = impl::mfma<MI>(nothing, nothing, acc_t{});
    }

    // Prologue.  Tile indices past the end are clamped to the last tile (a redundant, in-bounds
    // load whose data is never used), which keeps the main loop free of branches.
    //   register-staged: K-tile 0 into LDS stage 0, K-tile 1 into the staging registers
    //   direct-to-LDS  : K-tiles 0 .. NS-2 on their way into stages 0 .. NS-2; wait for tile 0
    const int last_tile = ntiles - 1;
    // loads that may still be in flight when a tile is needed: those of the NS - 2 tiles after it
    // (the wait counter holds 6 bits: a deeper ring than that waits for more than it must)
    constexpr int IN_FLIGHT = DTL ? ((NS - 2) * (CX + CY) < 64 ? (NS - 2) * (CX + CY) : 63) : 0;
    // K-tile t sits in stage (first_stage + t) % NS, with first_stage chosen so that the K-tiles
    // left after the first ntiles % NS of them start in stage 0 (see the main loop).
    const int peeled      = ntiles % NS;
    const int first_stage = peeled == 0 ? 0 : NS - peeled;
    auto      stage_after = [](int stage, int n) { // (stage + n) % NS for 0 <= n < NS
        const int u = stage + n;
        return u >= NS ? u - NS : u;
    };
    if constexpr(DTL)
    {
        impl::static_for<0, NS - 1>([&](auto s_c) {
            constexpr int s     = decltype(s_c)::value;
            const int     stage = stage_after(first_stage, s);
            impl::static_for<0, CX + CY>(
                [&](auto i) { dma_item(decltype(i)::value, min(s, last_tile), stage, std::true_type{}); });
        });
        impl::ring_barrier<IN_FLIGHT>();
    }
    else
    {
        impl::static_for<0, CX + CY>([&](auto i) { load_item(decltype(i)::value, 0); });
        impl::static_for<0, CX + CY>([&](auto i) { store_item(decltype(i)::value, first_stage, 0, std::true_type{}); });
        impl::static_for<0, CX + CY>([&](auto i) { load_item(decltype(i)::value, min(1, last_tile)); });
        __syncthreads();
    }
    impl::static_for<0, NRX + NRY>([&](auto q) { read_item(decltype(q)::value, 0, first_stage, 0); });
#if defined(ROCM_SGEMM_PHASE_STAMPS)
    stamp_loop_begin = wall_clock64();
    stamp_cycles     = clock64();
#endif

    // Main loop: one barrier per K-tile, and a software pipeline written out slot by slot.
    //
    // A wave issues in order, and an MFMA holds the matrix pipe for 64 (32x32x2) or 32 (16x16x4)
    // cycles, so between two MFMAs there is room for a few other instructions but a long run of
    // them leaves the pipe idle.  Every k-block therefore issues its 4*TM*TN MFMAs one per "slot",
    // and each slot carries at most a few items of data movement; the scheduling fence after every
    // slot keeps the compiler from clustering them again.  In iteration t (K-tile t in stage cur):
    //   every k-block but the last : reads the fragments of the next k-block
    //   k-block 0, register-staged : alternately stores one staged chunk of K-tile t+1 into the
    //                                other LDS stage (its last readers all passed the previous
    //                                barrier) and reloads that register with the same chunk of
    //                                K-tile t+2
    //   k-block 0, direct-to-LDS   : issues the loads of K-tile t+NS-1 into the stage that K-tile
    //                                t-1 occupied (same argument)
    //   last k-block               : barrier in slot 0 (direct-to-LDS: after waiting for this
    //                                wave's loads of K-tile t+1 only, the later ones stay in
    //                                flight), then reads the first fragments of K-tile t+1
    constexpr int SLOTS = 4 * TM * TN;
    constexpr int NR    = NRX + NRY;
    constexpr int NMOVE = DTL ? CX + CY : 2 * (CX + CY);
    // Slot assignment.  Reads of a k-block are spread over READ_SPAN slots starting at slot 0 (at
    // the barrier slot in the last k-block); the movement items of the K-tile are spread over
    // the MOVE_KBS first k-blocks.
    constexpr int BARRIER_SLOT = 0; // slot of the last k-block that carries the barrier
    // Single-float loads are four times as many.  A ring of three or more stages has a whole
    // K-tile of slack, so they are spread over all k-blocks but the last; with two stages a load
    // must land before this iteration's barrier, so they are issued as early as two per slot allow.
    constexpr int DENSE_KBS    = impl::max_int(1, (NMOVE + 2 * SLOTS - 1) / (2 * SLOTS));
    constexpr int MOVE_KBS     = (DTL && (DGX == 1 || DGY == 1)) ? (NS >= 3 || DENSE_KBS > NKB - 1 ? NKB - 1 : DENSE_KBS)
                                                    : 1;
    constexpr int MOVE_SLOTS   = MOVE_KBS * SLOTS;
    // One K-tile of the pipeline: K-tile t sits in stage `cur_c`.  With `ragged_c` false the caller
    // guarantees that every K-tile touched here (t + 1, and the one being fetched) is a whole one
    // before the last, so nothing is clamped or masked.
    auto k_tile_step = [&](int t, auto cur_c, auto ragged_c) {
        constexpr bool ragged     = decltype(ragged_c)::value;
        const int      cur        = cur_c; // stage of K-tile t
        const int      nxt        = cur == NS - 1 ? 0 : cur + 1; // stage of K-tile t + 1
        const int      fill_stage = cur == 0 ? NS - 1 : cur - 1; // stage of K-tile t + NS - 1
        const int      fill_tile  = ragged ? min(t + (DTL ? NS - 1 : 2), last_tile) : t + (DTL ? NS - 1 : 2);
        impl::static_for<0, NKB>([&](auto kb_c) {
            constexpr int  kb       = decltype(kb_c)::value;
            constexpr int  slot     = kb & 1;
            constexpr bool last_kb  = kb == NKB - 1;
            constexpr int  read_off = last_kb ? BARRIER_SLOT : 0;
            constexpr int  read_span
                = impl::max_int(1, SLOTS - read_off); // reads spread over the rest of the k-block
            impl::static_for<0, SLOTS>([&](auto m_c) {
                constexpr int m = decltype(m_c)::value;
                constexpr int r = m / (TM * TN);
                constexpr int i = (m / TN) % TM;
                constexpr int j = m % TN;
                if constexpr(last_kb && m == BARRIER_SLOT)
                {
                    if constexpr(DTL)
                        impl::ring_barrier<IN_FLIGHT>();
                    else
                        __syncthreads();
                }
                // reads whose slot is m: read e sits in slot read_off + e * read_span / NR
                constexpr int rb = impl::items_before(m - read_off, read_span, NR);
                constexpr int re = impl::items_before(m - read_off + 1, read_span, NR);
                impl::static_for<rb, re>([&](auto e_c) {
                    constexpr int e = decltype(e_c)::value;
                    if constexpr(last_kb)
                        read_item(e, slot ^ 1, nxt, 0);
                    else
                        read_item(e, slot ^ 1, cur, kb + 1);
                });
                // movement items whose (k-block, slot) is (kb, m): item g sits at position
                // g * MOVE_SLOTS / NMOVE of the first MOVE_KBS k-blocks
                if constexpr(kb < MOVE_KBS)
                {
                    constexpr int gb = impl::items_before(kb * SLOTS + m, MOVE_SLOTS, NMOVE);
                    constexpr int ge = impl::items_before(kb * SLOTS + m + 1, MOVE_SLOTS, NMOVE);
                    impl::static_for<gb, ge>([&](auto g_c) {
                        constexpr int g = decltype(g_c)::value;
                        if constexpr(DTL)
                            dma_item(g, fill_tile, fill_stage, ragged_c);
                        else if constexpr(g % 2 == 0)
                            store_item(g / 2, nxt, t + 1, ragged_c);
                        else
                            load_item(g / 2, fill_tile);
                    });
                }
                acc[i][j] = impl::mfma<MI>(fx[slot][i][r], fy[slot][j][r], acc[i][j]);
                __builtin_amdgcn_sched_barrier(0);
            });
        });
    };
    // Keeps the accumulators in the accumulation registers across the boundaries between the loops
    // below (an empty asm with a register-class constraint: no instruction).  Without it the
    // register allocator moves accumulators to ordinary registers and back at those boundaries.
    auto pin_acc = [&]() { // not a generic lambda: the asm operand must name `acc` directly
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
        for(int i = 0; i < TM; ++i)
#pragma unroll
            for(int j = 0; j < TN; ++j)
                asm volatile("" : "+a"(acc[i][j]));
#endif
    };
    // Steady state: NS K-tiles per trip, so that every stage index is a constant.  The LDS address
    // of every fragment read and the LDS target of every load are then loop-invariant (a register
    // set up once, plus an immediate offset) and the loop holds no vector-ALU instruction at all.
    // That matters more than it looks: on this part a vector-ALU instruction issued into a stream
    // of back-to-back MFMAs holds up the next MFMA by about 13 cycles (scalar instructions, LDS
    // reads, direct-to-LDS loads and barriers cost nothing there), and a loop that computes
    // `stage offset + lane offset` for its reads spends six of them per K-tile.
    // The ntiles % NS K-tiles that do not fill a trip come first, one at a time with the stage in
    // a register; the prologue has placed K-tile 0 so that the first whole trip starts in stage 0.
    pin_acc();
    {
        int stage = first_stage;
        for(int t = 0; t < peeled; ++t)
        {
            k_tile_step(t, stage, std::true_type{});
            stage = stage_after(stage, 1);
        }
    }
    pin_acc();
    if constexpr(!EDGE)
    {
        // nothing to mask; the clamp of the tile index is one scalar instruction per K-tile
        for(int t = peeled; t < ntiles; t += NS)
        {
            impl::static_for<0, NS>([&](auto s_c) { k_tile_step(t + decltype(s_c)::value, s_c, std::true_type{}); });
        }
    }
    else
    {
        // Only the last trip touches the last K-tile (it fetches it, or multiplies it): the trips
        // before it run without the masks of a ragged depth, whose compares and selects are
        // vector-ALU instructions, two per load.
        int t = peeled;
        for(; t + 2 * NS <= ntiles; t += NS)
        {
            impl::static_for<0, NS>([&](auto s_c) { k_tile_step(t + decltype(s_c)::value, s_c, std::false_type{}); });
        }
        pin_acc();
        if(t < ntiles)
        {
            impl::static_for<0, NS>([&](auto s_c) { k_tile_step(t + decltype(s_c)::value, s_c, std::true_type{}); });
        }
    }
#if defined(ROCM_SGEMM_PHASE_STAMPS)
    stamp_loop_end = wall_clock64();
    stamp_cycles   = clock64() - stamp_cycles;
#endif
    if constexpr(DTL)
    {
        // the clamped loads of the last iterations still target this workgroup's LDS
        impl::wait_all_loads();
    }

    // Epilogue: accumulator register v of lane (h, c) holds MFMA row acc_row(v, h), column c.
    // Destination: the output matrix, or this slice's packed rows x cols partial (split-K), or this
    // segment's BM x BN partial tile (stream-K tail; tile-local coordinates, never clipped).
    // The accumulators are stored as they are (straight from the accumulation registers); a call
    // with alpha != 1 or beta != 0 points P at a workspace and lets the reduction kernel blend.
    // The store addresses depend only on the lane, so the compiler would compute them once, ahead
    // of the segment loop, and keep them in registers through the main loop; passing the lane
    // coordinates through an empty asm here pins that arithmetic to the epilogue.
    int h_e = h, c_e = c;
#if defined(__HIP_DEVICE_COMPILE__)
    asm volatile("" : "+v"(h_e), "+v"(c_e));
#endif
    // Where a tile goes or comes from: base, row stride, origin of the macro tile, matrix extent.
    struct tile_place
    {
        float* base;
        int    ld, row0, col0, row_end, col_end;
    };
    const bool       to_partial = tail || args.split_k > 1;
    const tile_place result{args.P + batch * args.stride_p, args.ldp, m0, n0, args.rows, args.cols};
    // the partial of split-K slice s (tiles at their place in a packed rows x cols matrix)
    auto slice_place = [&](int s) {
        return tile_place{args.partial
                              + (static_cast<size_t>(batch) * args.split_k + s) * args.rows * static_cast<size_t>(args.cols),
                          args.cols, m0, n0, args.rows, args.cols};
    };
    // the partial tile of segment s of tail workgroup g (never clipped)
    auto segment_place = [&](int g, int s) {
        return tile_place{args.partial + (static_cast<size_t>(g) * 2 + s) * (BM * BN), BN, 0, 0, BM, BN};
    };
    const tile_place mine = tail ? segment_place(tail_g, seg) : (args.split_k > 1 ? slice_place(slice) : result);

    // Plain stores of one row of MFMA tiles: `vals[j][v]` is accumulator register v of tile (i, j),
    // v in [v_begin, v_begin + v_count); 128-bit where the lane's values are adjacent.
    auto put_row = [&](const tile_place& t, int i, auto& vals, auto v_begin_c, auto v_count_c) {
#pragma unroll
        for(int v = decltype(v_begin_c)::value; v < decltype(v_begin_c)::value + decltype(v_count_c)::value; ++v)
        {
            const int mi  = impl::acc_row<MI>(v, h_e);
            const int row = t.row0 + wm0 + impl::tile_index<X_KC, VM, MI>(i, mi);
            if(EDGE && row >= t.row_end)
            {
                continue;
            }
            float* prow = t.base + static_cast<size_t>(row) * t.ld;
            if constexpr(!Y_KC && VN > 1)
            {
#pragma unroll
                for(int g = 0; g < TN / VN; ++g)
                {
                    const int col = t.col0 + wn0 + g * MI * VN + VN * c_e;
                    if constexpr(VN == 4)
                    {
                        const f32x4 o = {vals[g * 4 + 0][v], vals[g * 4 + 1][v], vals[g * 4 + 2][v], vals[g * 4 + 3][v]};
                        if constexpr(!EDGE)
                        {
                            *reinterpret_cast<f32x4*>(prow + col) = o;
                        }
                        else if(col + 3 < t.col_end)
                        {
                            *reinterpret_cast<f32x4_e*>(prow + col) = o;
                        }
                        else
                        {
                            if(col < t.col_end) prow[col] = o.x;
                            if(col + 1 < t.col_end) prow[col + 1] = o.y;
                            if(col + 2 < t.col_end) prow[col + 2] = o.z;
                        }
                    }
                    else
                    {
                        const f32x2 o = {vals[g * 2 + 0][v], vals[g * 2 + 1][v]};
                        if constexpr(!EDGE)
                        {
                            *reinterpret_cast<f32x2*>(prow + col) = o;
                        }
                        else if(col + 1 < t.col_end)
                        {
                            *reinterpret_cast<f32x2_e*>(prow + col) = o;
                        }
                        else if(col < t.col_end)
                        {
                            prow[col] = o.x;
                        }
                    }
                }
            }
            else
            {
                // one column per tile: tile j of this lane is column MI * j + c of the wave tile
                static_assert(impl::tile_index<Y_KC, VN, MI>(1, 0) == MI || TN == 1, "tiles are stacked here");
                float* const pcol = prow + (t.col0 + wn0 + c_e);
                impl::static_for<0, TN>([&](auto j_c) {
                    constexpr int j = decltype(j_c)::value;
                    if(!EDGE || t.col0 + wn0 + c_e + MI * j < t.col_end)
                    {
#if defined(__HIP_DEVICE_COMPILE__)
                        if constexpr(std::is_same_v<std::remove_reference_t<decltype(vals)>, acc_t[TN]>)
                        {
                            // straight from the accumulation register: left to itself the compiler
                            // may first copy all accumulators of the wave into ordinary registers
                            // (operands are locals of this lambda: an asm statement in a generic
                            // lambda cannot name what it captures)
                            float* const where = pcol;
                            const float  what  = vals[j][v];
                            asm volatile("global_store_dword %0, %1, off offset:%2" ::"v"(where), "a"(what), "n"(MI * j * 4)
                                         : "memory");
                        }
                        else
#endif
                        {
                            pcol[MI * j] = vals[j][v];
                        }
                    }
                });
            }
        }
    };

    // Traffic between workgroups of one launch (the parts of a tile that is summed in the launch):
    //   SHARE    stores other workgroups' waves will read: written through to memory, never left
    //            dirty in this XCD's L2
    //   FETCH    value  = what another workgroup shared: never a line a cache still holds from before
    //   GATHER   value += the same
    // These are buffer accesses with the agent-scope cache policy (the bits agent-scope atomic loads
    // and stores carry): one 32-bit offset per element from a wave-uniform base, elements outside
    // the matrix get an offset the range check rejects (their stores are dropped, their loads
    // return zero), so the code has no branches.  Offsets stay below 2 GiB (the host checks).
    constexpr int SHARE = 1, FETCH = 2, GATHER = 3;
    constexpr int agent_scope = 16; // cache policy bit sc1
    auto coherent = [](auto mode_c, __amdgpu_buffer_rsrc_t rsrc, int byte_offset, float value) -> float {
        constexpr int mode = decltype(mode_c)::value;
#if defined(__HIP_DEVICE_COMPILE__)
        if constexpr(mode == SHARE)
        {
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, value), rsrc, byte_offset, 0, agent_scope);
            return value;
        }
        else
        {
            const float got = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, agent_scope));
            return mode == FETCH ? got : value + got;
        }
#else
        (void)rsrc, (void)byte_offset;
        return value;
#endif
    };
    auto descriptor = [](const tile_place& t) {
        return __builtin_amdgcn_make_buffer_rsrc(t.base, 0, 0x7FFFFFFF, 0x00020000);
    };
    constexpr int rejected = static_cast<int>(0x80000000u); // beyond any buffer declared above
    auto coherent_row = [&](auto mode_c, const tile_place& t, int i, auto& vals, auto v_begin_c, auto v_count_c) {
        constexpr int                mode = decltype(mode_c)::value;
        const __amdgpu_buffer_rsrc_t rsrc = descriptor(t);
#pragma unroll
        for(int v = decltype(v_begin_c)::value; v < decltype(v_begin_c)::value + decltype(v_count_c)::value; ++v)
        {
            const int  row    = t.row0 + wm0 + impl::tile_index<X_KC, VM, MI>(i, impl::acc_row<MI>(v, h_e));
            const bool row_ok = !EDGE || row < t.row_end;
#pragma unroll
            for(int j = 0; j < TN; ++j)
            {
                const int   col = t.col0 + wn0 + impl::tile_index<Y_KC, VN, MI>(j, c_e);
                const int   off = row_ok && (!EDGE || col < t.col_end) ? (row * t.ld + col) * 4 : rejected;
                const float got = coherent(mode_c, rsrc, off, vals[j][v]);
                if constexpr(mode >= FETCH) vals[j][v] = got;
            }
#if defined(__HIP_DEVICE_COMPILE__)
            // keeps the offsets of later rows from being computed (and held in registers) up front
            __builtin_amdgcn_sched_barrier(0);
#endif
        }
    };
    // With waves along K the lane's share is `summed` instead: four adjacent columns of NSUM rows
    // of the tile the workgroup has added up from the replicas' images.
    constexpr int NSUM = WK > 1 ? BM * BN / 4 / NT : 1;
    f32x4         summed[NSUM];
    auto          put_summed = [&](const tile_place& t) {
#pragma unroll
        for(int g = 0; g < NSUM; ++g)
        {
            const int p   = (g * NT + tid) * 4; // where the image held the values (see EX_ROW_BIT)
            const int l   = p ^ ((((p / BN) >> Cfg::EX_ROW_BIT) & 1) << 5);
            const int row = t.row0 + l / BN;
            const int col = t.col0 + l % BN;
            float*    dst = t.base + static_cast<size_t>(row) * t.ld + col;
            if constexpr(!EDGE)
            {
                *reinterpret_cast<f32x4*>(dst) = summed[g];
            }
            else if(row < t.row_end)
            {
                if(col + 3 < t.col_end)
                {
                    *reinterpret_cast<f32x4_e*>(dst) = summed[g];
                }
                else
                {
                    if(col < t.col_end) dst[0] = summed[g].x;
                    if(col + 1 < t.col_end) dst[1] = summed[g].y;
                    if(col + 2 < t.col_end) dst[2] = summed[g].z;
                }
            }
        }
    };
    auto coherent_summed = [&](auto mode_c, const tile_place& t) {
        constexpr int                mode = decltype(mode_c)::value;
        const __amdgpu_buffer_rsrc_t rsrc = descriptor(t);
#pragma unroll
        for(int g = 0; g < NSUM; ++g)
        {
            const int  p      = (g * NT + tid) * 4; // where the image held the values (see EX_ROW_BIT)
            const int  l      = p ^ ((((p / BN) >> Cfg::EX_ROW_BIT) & 1) << 5);
            const int  row    = t.row0 + l / BN;
            const int  col    = t.col0 + l % BN;
            const bool row_ok = !EDGE || row < t.row_end;
#pragma unroll
            for(int e = 0; e < 4; ++e)
            {
                const int   off = row_ok && (!EDGE || col + e < t.col_end) ? (row * t.ld + col + e) * 4 : rejected;
                const float got = coherent(mode_c, rsrc, off, summed[g][e]);
                if constexpr(mode >= FETCH) summed[g][e] = got;
            }
        }
    };
    // The lane's whole share: plain stores, or stores for other workgroups to read.
    auto put_tile = [&](const tile_place& t) {
        if constexpr(WK > 1)
            put_summed(t);
        else
        {
#if defined(__HIP_DEVICE_COMPILE__)
            // put_row may store accumulation registers through asm statements, whose operands the
            // compiler's hazard recogniser does not see: a store must not read a register within 18
            // wait states of the MFMA that wrote it.  Volatile asm statements keep their order.
            asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#endif
            impl::static_for<0, TM>([&](auto i_c) {
                put_row(t, decltype(i_c)::value, acc[decltype(i_c)::value], std::integral_constant<int, 0>{},
                        std::integral_constant<int, ACC>{});
            });
        }
    };
    auto share_tile = [&](const tile_place& t) {
        if constexpr(WK > 1)
            coherent_summed(std::integral_constant<int, SHARE>{}, t);
        else
            impl::static_for<0, TM>([&](auto i_c) {
                coherent_row(std::integral_constant<int, SHARE>{}, t, decltype(i_c)::value, acc[decltype(i_c)::value],
                             std::integral_constant<int, 0>{}, std::integral_constant<int, ACC>{});
            });
    };
    // The sum of the parts `place(n)`, n = 0 .. count - 1, added in that order, stored to the
    // result.  The sums live in registers of their own: arithmetic on the accumulators would pull
    // them out of the accumulation registers for the whole kernel.
    auto sum_parts = [&](int count, auto&& place) {
        if constexpr(WK > 1)
        {
            coherent_summed(std::integral_constant<int, FETCH>{}, place(0));
            for(int n = 1; n < count; ++n)
                coherent_summed(std::integral_constant<int, GATHER>{}, place(n));
            put_summed(result);
        }
        else
        {
            // about 32 values of the lane at a time: enough loads in flight, few registers
            constexpr int VCH = impl::max_int(1, (32 / TN < ACC ? 32 / TN : ACC));
            impl::static_for<0, TM*(ACC / VCH)>([&](auto n_c) {
                constexpr int                          i = decltype(n_c)::value / (ACC / VCH);
                const std::integral_constant<int, (decltype(n_c)::value % (ACC / VCH)) * VCH> v0;
                const std::integral_constant<int, VCH>                                         vn;
                acc_t                                  sum[TN];
                coherent_row(std::integral_constant<int, FETCH>{}, place(0), i, sum, v0, vn);
                for(int n = 1; n < count; ++n)
                    coherent_row(std::integral_constant<int, GATHER>{}, place(n), i, sum, v0, vn);
                put_row(result, i, sum, v0, vn);
            });
        }
    };

    if constexpr(WK > 1)
    {
        // Waves along K: every replica of the wave grid holds a partial of the whole macro tile.
        // Each leaves it in LDS as a row-major BM x BN image; then the workgroup sums the images in
        // replica order (fixed, so the result does not depend on timing); a thread keeps four
        // adjacent columns of NSUM rows.
        // linear index of element (r, n) of an image, bank-swizzled (tile_config::EX_ROW_BIT)
        auto image_index = [](int r, int n) { return (r * BN + n) ^ (((r >> Cfg::EX_ROW_BIT) & 1) << 5); };
        __syncthreads(); // every wave is done with the stages: the images reuse their memory
        float* image = lds + wk * (BM * BN);
#pragma unroll
        for(int i = 0; i < TM; ++i)
#pragma unroll
            for(int v = 0; v < ACC; ++v)
            {
                const int r = wm0 + impl::tile_index<X_KC, VM, MI>(i, impl::acc_row<MI>(v, h_e));
                if constexpr(!Y_KC && VN > 1)
                {
                    // a lane's VN tiles are adjacent columns: one 64- or 128-bit write, contiguous
                    // across the lanes
#pragma unroll
                    for(int g = 0; g < TN / VN; ++g)
                    {
                        float* dst = image + image_index(r, wn0 + g * MI * VN + VN * c_e);
                        if constexpr(VN == 4)
                            *reinterpret_cast<f32x4*>(dst)
                                = f32x4{acc[i][g * 4 + 0][v], acc[i][g * 4 + 1][v], acc[i][g * 4 + 2][v], acc[i][g * 4 + 3][v]};
                        else
                            *reinterpret_cast<f32x2*>(dst) = f32x2{acc[i][g * 2 + 0][v], acc[i][g * 2 + 1][v]};
                    }
                }
                else
                {
#pragma unroll
                    for(int j = 0; j < TN; ++j)
                        image[image_index(r, wn0 + impl::tile_index<Y_KC, VN, MI>(j, c_e))] = acc[i][j][v];
                }
            }
        __syncthreads();
#pragma unroll
        for(int g = 0; g < NSUM; ++g)
        {
            const int p = (g * NT + tid) * 4; // linear position: consecutive threads, consecutive banks
            f32x4     o = *reinterpret_cast<const f32x4*>(lds + p);
#pragma unroll
            for(int w = 1; w < WK; ++w)
                o += *reinterpret_cast<const f32x4*>(lds + w * (BM * BN) + p);
            summed[g] = o;
        }
    }

    // (Only kernels of at most four waves that each own at most a 64 x 64 share of the tile can sum
    // in the launch: with a larger share one wave would have too much to add up, and the code
    // would not fit next to 128 or 256 accumulators without spilling.  The host never passes
    // counters to the others.)
    if(!Cfg::SUMS_IN_LAUNCH || !to_partial || args.counters == nullptr)
    {
        // the tile is final, or a second kernel sums the partial tiles
        put_tile(mine);
    }
    else if constexpr(Cfg::SUMS_IN_LAUNCH)
    {
        // Partial tile, summed in this launch.  Every wave shares its part of the tile, then takes
        // a ticket from the counter of (tile, wave position); the wave that draws the last ticket
        // knows that every other part is complete in memory, adds them all up in a fixed order -
        // K slices in slice order, tail segments in workgroup order - and stores the result.  No
        // wave ever waits for another.
        // Ordering.  Writers: the parts are stored with the agent-scope cache policy (written through,
        // never left dirty in this XCD's L2), and the wave then waits until every one of those
        // stores has been acknowledged (s_waitcnt vmcnt(0): on this target stores count in vmcnt
        // like loads) before it draws the ticket.  A wave's stores and its atomic go to different
        // memory channels and are ordered at issue only, so without that wait the ticket could
        // become visible before a part has landed.  The workgroup-scope fences emit no
        // instruction here; they only keep the compiler from moving memory accesses across the
        // ticket.  Reader: the parts are read with the same cache policy by loads that are issued
        // after the ticket has come back (the branch below depends on its value), so no cache can
        // hand out a line that is older than the ticket.
        share_tile(mine);
        impl::wait_all_loads();
        const int tile_id  = tail ? tail_u0 + seg : wg; // tail: number of the tail tile; else the tile
        const int expected = tail ? min(((tile_id + 1) * k_tiles - 1) / args.tail_per, args.tail_groups - 1)
                                        - (tile_id * k_tiles) / args.tail_per + 1
                                  : args.split_k;
        unsigned* counter = args.counters
                            + (static_cast<size_t>(batch) * (tail ? tiles - args.tail_begin : tiles) + tile_id) * (NT / 64)
                            + wave;
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        unsigned ticket = 0;
        if(lane == 0)
        {
            ticket = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        ticket = __builtin_amdgcn_readfirstlane(ticket);
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        if(static_cast<int>(ticket) == expected - 1)
        {
            if(lane == 0)
            {
                // left at zero for the next launch that uses the counter (stream order separates them)
                __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if(tail)
            {
                const int g_first = (tile_id * k_tiles) / args.tail_per;
                sum_parts(expected, [&](int n) {
                    const int g = g_first + n;
                    return segment_place(g, (g * args.tail_per) / k_tiles == tile_id ? 0 : 1);
                });
            }
            else
            {
                sum_parts(args.split_k, slice_place);
            }
        }
    }
    if(seg + 1 < nseg)
    {
        // the next segment refills the LDS stages: every wave must be done reading them
        __syncthreads();
    }
    } // segments
#if defined(ROCM_SGEMM_PHASE_STAMPS) && defined(__HIP_DEVICE_COMPILE__)
    __builtin_amdgcn_s_waitcnt(0); // the stores have completed
    if(args.stamps != nullptr && lane == 0)
    {
        unsigned long long* out
            = args.stamps + ((static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * (NT / 64) + wave) * 8;
        out[0] = stamp_start;
        out[1] = stamp_loop_begin;
        out[2] = stamp_loop_end;
        out[3] = wall_clock64();
        out[4] = stamp_cycles;
        out[5] = __builtin_amdgcn_s_getreg((31 << 11) | 20) & 7; // XCC_ID
    }
#endif
}

} // namespace kernel
} // namespace rocm_sgemm

#endif
