/*
 * rocm_sgemm.h - flat C ABI of the MI355X (gfx950) SGEMM library.
 *
 * This is the seam every binding goes through (C++ templates in <rocm_sgemm/gemm.hpp>, Python
 * ctypes, the tuner's trial binary).  Plain pointers and sizes only; the stream is passed as the
 * opaque hipStream_t value (a pointer), NULL meaning the default stream.
 *
 * All matrices are dense and packed, exactly as in the reference API
 * (reference rocm_sgemm/include/rocm_sgemm/gemm.hpp:33-52, common/matrix.hpp:130-139):
 *   row-major X (r x c): element (i, j) at i * c + j      column-major: at j * r + i
 *   A is M x K, B is K x N, C is M x N;  C <- A * B  (alpha = 1, beta = 0, C overwritten).
 * A, B, C are device pointers owned by the caller.  Calls only enqueue work on `stream`; they do
 * not synchronise.  Calls are re-entrant and may come from several threads.  The only state the
 * library keeps is one workspace buffer per (device, stream) that ever ran a problem needing one
 * (split-K, stream-K tail, alpha / beta): it is grown on demand and reused by later calls on that
 * stream, which execute in order; rocm_sgemm_release_workspaces() gives the memory back.
 */
#ifndef ROCM_SGEMM_C_H
#define ROCM_SGEMM_C_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Same enumerator order as rocm_sgemm::m_layout (reference kernel/common.hpp:36-40). */
enum
{
    ROCM_SGEMM_ROW_MAJOR = 0,
    ROCM_SGEMM_COL_MAJOR = 1
};

enum
{
    ROCM_SGEMM_STATUS_OK            = 0,
    ROCM_SGEMM_STATUS_INVALID_ARG   = 1, /* null pointer, zero or > INT_MAX dimension, bad layout */
    ROCM_SGEMM_STATUS_NO_KERNEL     = 2, /* no compiled kernel for the requested tile shape:
                                            the condition under which the reference throws
                                            std::runtime_error (kernel_launcher.hpp:89-94) */
    ROCM_SGEMM_STATUS_LAUNCH_FAILED = 3, /* HIP refused the launch or the workspace allocation */
    ROCM_SGEMM_STATUS_BAD_CONFIG    = 4, /* config fields out of range */
    ROCM_SGEMM_STATUS_WORKSPACE_TOO_LARGE = 5 /* rocm_sgemm_f32_no_alloc only: the problem's
                                                 partial products do not fit the fixed scratch */
};

/* Size of the fixed device scratch array behind rocm_sgemm_f32_no_alloc, per GPU. */
#define ROCM_SGEMM_NO_ALLOC_SCRATCH_BYTES (128u * 1024u * 1024u)

/*
 * Tuned launch parameters of one table entry.  Takes the place of the reference's 9-int tuple
 * (block_size, block_m, block_n, block_k, warp_tile_*, thread_tile_*, threads_n;
 * reference config/gemm_config.json:14-24), re-parameterised for MFMA:
 *   macro_m x macro_n : output tile of one workgroup (in terms of the caller's M and N)
 *   k_tile            : depth staged through LDS per pipeline step
 *   waves_m x waves_n : wave64 grid inside the workgroup (block size = 64 * waves_m * waves_n)
 *   mfma              : 32 = v_mfma_f32_32x32x2_f32, 16 = v_mfma_f32_16x16x4_f32
 *   stages            : how a K-tile travels from HBM to LDS.  0 = through registers into two LDS
 *                       stages; n >= 2 = straight into a ring of n LDS stages
 *                       (buffer_load ... lds): 16 bytes per lane when the operand lines are
 *                       16-byte aligned (pointers, leading dimensions, and K under an operand
 *                       stored K-contiguous), else 4 bytes per lane, which needs no alignment;
 *                       ragged edges are masked in either case
 *   split_k           : number of K slices summed by a second kernel (1 = none)
 *   group_m           : height, in tiles, of the bands of the XCD-aware tile order
 *   wave_slots        : workgroups the GPU runs at once, used by the stream-K tail: the K range of
 *                       the tiles of a short last wave is dealt out evenly to all those slots
 *                       (partial tiles summed by a second kernel) so that every CU has work.
 *                       0 = ask the runtime (CUs x occupancy), 1 = never, n > 1 = assume n
 *                       (tuning / testing aid)
 *   waves_k           : replicas of the waves_m x waves_n wave grid along K (0 or 1 = none).
 *                       Replica w multiplies the w-th part of every K-tile over the whole wave
 *                       tile, and the partial tiles are summed through LDS before the store:
 *                       a small macro tile (many tiles for 256 CUs) keeps a large wave tile.
 *                       Block size = 64 * waves_m * waves_n * waves_k.  Part of the tile shape,
 *                       like macro_m .. stages
 *   partial_sums      : who adds up the partial tiles of a K split or a stream-K tail.
 *                       1 = a second kernel; 2 = the GEMM launch itself, whenever it can (the wave
 *                       that completes a tile's counter adds the tile's parts up: no second
 *                       launch, but one wave reads all parts of its share of the tile);
 *                       0 = the library decides, which at present means a second kernel: with
 *                       the wait for its write-through stores that the scheme needs, the launch
 *                       lost to the second kernel on every problem it was timed on.
 *                       The result is the same bit for bit either way (same order of addition)
 */
typedef struct rocm_sgemm_config
{
    int macro_m;
    int macro_n;
    int k_tile;
    int waves_m;
    int waves_n;
    int mfma;
    int stages;
    int split_k;
    int group_m;
    int wave_slots;
    int waves_k;
    int partial_sums;
} rocm_sgemm_config;

/*
 * C <- A * B.  Replaces rocm_sgemm::gemm<layout_C, layout_A, layout_B, float>
 * (reference rocm_sgemm/src/gemm.cpp:8-41): picks the tuned config for (M, N, K, layouts) and
 * launches one kernel (two when the config splits K) on `stream`.
 * Returns a ROCM_SGEMM_STATUS_* value; rocm_sgemm_last_error() describes a failure.
 */
int rocm_sgemm_f32(int          layout_c,
                   int          layout_a,
                   int          layout_b,
                   float*       C,
                   const float* A,
                   const float* B,
                   size_t       M,
                   size_t       N,
                   size_t       K,
                   void*        stream);

/*
 * The same product as rocm_sgemm_f32 - same config, same kernels, same bits - for callers that
 * cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference (whose kernels never need a
 * workspace).  rocm_sgemm_f32 keeps the partial products of a split-K or stream-K-tail config in
 * a workspace it allocates; this entry point keeps them in a fixed array of
 * ROCM_SGEMM_NO_ALLOC_SCRATCH_BYTES of device memory that is part of the library's code object
 * (every GPU the library runs on holds it until the process ends) and calls no hipMalloc, hipFree
 * or other allocating routine.  A problem whose partial products need more than that is refused
 * with ROCM_SGEMM_STATUS_WORKSPACE_TOO_LARGE and nothing is enqueued (a product of any size whose
 * config neither splits K nor deals out a tail needs no scratch and always runs).
 * All calls on one GPU share the array: two calls may not overlap in time on one GPU (calls on
 * one stream never do; calls on different streams, or replays of graphs that recorded such
 * calls, must be ordered by the caller).  Nothing in the array needs clearing between calls:
 * every partial product a call reads it has written itself.
 */
int rocm_sgemm_f32_no_alloc(int          layout_c,
                            int          layout_a,
                            int          layout_b,
                            float*       C,
                            const float* A,
                            const float* B,
                            size_t       M,
                            size_t       N,
                            size_t       K,
                            void*        stream);

/*
 * Bytes of workspace rocm_sgemm_f32 would use for the partial products of this problem under the
 * config it plans (0: the plan neither splits K nor deals out a stream-K tail); what
 * rocm_sgemm_f32_no_alloc compares with ROCM_SGEMM_NO_ALLOC_SCRATCH_BYTES.  Host only: nothing is
 * allocated, launched or read.  No counterpart in the reference, which never splits K
 * (rocm_sgemm/src/gemm.cpp:21-25: one block per output tile).
 */
int rocm_sgemm_workspace_bytes(int layout_c, int layout_a, int layout_b, size_t M, size_t N, size_t K, size_t* bytes);

/*
 * Same product with an explicit config instead of the table lookup.  Replaces the tuner's
 * per-trial hipRTC compile-and-launch (reference rocm_sgemm/config/tuner.cpp:183-216,386-438):
 * every tile shape of the search space is precompiled, so a trial is just this call.
 */
int rocm_sgemm_f32_with_config(const rocm_sgemm_config* config,
                               int                      layout_c,
                               int                      layout_a,
                               int                      layout_b,
                               float*                   C,
                               const float*             A,
                               const float*             B,
                               size_t                   M,
                               size_t                   N,
                               size_t                   K,
                               void*                    stream);

/*
 * General form: for b in [0, batch_count)
 *     C_b <- alpha * A_b * B_b + beta * C_b,      Z_b = Z + b * stride_z (strides in elements).
 * lda / ldb / ldc are leading dimensions in elements: the distance between consecutive rows of a
 * row-major matrix or consecutive columns of a column-major one; 0 means packed (the reference's
 * layout).  beta == 0 never reads C.  alpha = 1, beta = 0, batch_count = 1 and packed operands is
 * exactly rocm_sgemm_f32.  The reference has no such entry: its bench only carries a batch_count
 * flag that scales buffers and flop counts while one product is launched
 * (reference benchmark/gemm/bench.cpp:49-51,72,77-85); this is the real batched launch, one grid
 * for all batches.  Batches must not overlap in C (stride_c >= one C matrix when batch_count > 1);
 * a stride of 0 broadcasts A or B.
 */
int rocm_sgemm_f32_strided_batched(int          layout_c,
                                   int          layout_a,
                                   int          layout_b,
                                   float        alpha,
                                   const float* A,
                                   size_t       lda,
                                   long long    stride_a,
                                   const float* B,
                                   size_t       ldb,
                                   long long    stride_b,
                                   float        beta,
                                   float*       C,
                                   size_t       ldc,
                                   long long    stride_c,
                                   size_t       M,
                                   size_t       N,
                                   size_t       K,
                                   size_t       batch_count,
                                   void*        stream);

/* Same with an explicit config (tests and tuning of the general form). */
int rocm_sgemm_f32_strided_batched_with_config(const rocm_sgemm_config* config,
                                               int                      layout_c,
                                               int                      layout_a,
                                               int                      layout_b,
                                               float                    alpha,
                                               const float*             A,
                                               size_t                   lda,
                                               long long                stride_a,
                                               const float*             B,
                                               size_t                   ldb,
                                               long long                stride_b,
                                               float                    beta,
                                               float*                   C,
                                               size_t                   ldc,
                                               long long                stride_c,
                                               size_t                   M,
                                               size_t                   N,
                                               size_t                   K,
                                               size_t                   batch_count,
                                               void*                    stream);

/*
 * Config lookup by the reference's rule (its generated detail::find_best_config,
 * reference rocm_sgemm/config/generate_config.py:174-267): exact (M, N, K, A, B, C) table hit,
 * else the entry with the same three layouts nearest in sum of squared log2 size ratios, else the
 * nearest entry of any layout, else the built-in default.  One refinement: among the same-layout
 * entries, those of the problem's own kind (M, N and K all multiples of 4, i.e. operand
 * lines 16-byte aligned in every layout, or not) are searched first, because the two
 * kinds run different kernels (16-byte vs 4-byte direct-to-LDS loads).  A second one: the table
 * that is searched holds, beside every tuned entry, its mirror image (N, M, K with the layouts of
 * A and B exchanged and all three flipped, macro_m / macro_n and waves_m / waves_n exchanged)
 * unless that problem was tuned itself: a column-major C is computed as C^T = B^T A^T, so the two
 * are one and the same launch, and an entry tuned in one layout serves two.  rocm_sgemm_table_entry
 * lists the tuned entries only.  Host-only, needs no GPU.
 */
int rocm_sgemm_nearest_config(size_t M, size_t N, size_t K, int layout_a, int layout_b, int layout_c,
                              rocm_sgemm_config* out);

/*
 * The config rocm_sgemm_f32 runs.  A table entry's own problem gets its entry.  Any other problem
 * starts from rocm_sgemm_nearest_config with the inherited split_k fitted to its own tile count
 * (dropped in favour of the stream-K tail when the grid would stay well under one workgroup per
 * CU, reduced when it would exceed four per CU); the cost model below then prices that config,
 * those of the next three nearest entries and the larger direct-to-LDS tile shapes of the family
 * at split_k 1, 2, 3, 4, 6 and 8, and the cheapest replaces the nearest entry's config if it is
 * expected to be at least 5 % faster (distance in log size says nothing about how a tile shape
 * divides M and N or how many tiles are left for 256 CUs).  Host-only, needs no GPU.
 */
int rocm_sgemm_find_config(size_t M, size_t N, size_t K, int layout_a, int layout_b, int layout_c,
                           rocm_sgemm_config* out);

/*
 * The same for `batch_count` products of one shape launched together, which is what
 * rocm_sgemm_f32_strided_batched runs: the tiles of all products fill the GPU together, so a batch
 * of small products wants larger tiles and less K splitting than one of them alone.  The table is
 * tuned on single products, so for batch_count > 1 no problem counts as a table entry.
 */
int rocm_sgemm_find_config_batched(size_t M, size_t N, size_t K, size_t batch_count, int layout_a, int layout_b,
                                   int layout_c, rocm_sgemm_config* out);

/*
 * The cost model used above: rough duration, in microseconds, of `batch_count` M x N x K products
 * launched together under `config` on MI355X (per tile the larger of matrix-pipe time at the wave-tile shape's sustained
 * efficiency and L2-to-LDS panel time, waves of tiles over 256 CUs, stream-K tail or K split
 * with their second pass, launch cost; constants fitted to tuner sweeps).  Good for ordering
 * configs.  No counterpart in the reference, whose lookup is by distance only.  Negative on
 * invalid arguments.
 */
double rocm_sgemm_predict_us(const rocm_sgemm_config* config, size_t M, size_t N, size_t K, size_t batch_count);

/* Number of entries in the tuned table (reference sorted_config_map), and entry `index` of it. */
int rocm_sgemm_table_size(void);
int rocm_sgemm_table_entry(int index, size_t* M, size_t* N, size_t* K, int* layout_a, int* layout_b,
                           int* layout_c, rocm_sgemm_config* out);

/*
 * The precompiled tile shapes (the tuner's search space).  Only macro_m .. stages and waves_k are
 * meaningful in `out`; split_k, group_m, wave_slots and partial_sums are launch-time parameters,
 * returned as 1, 4, 0 and 0.
 */
int rocm_sgemm_family_size(void);
int rocm_sgemm_family_entry(int index, rocm_sgemm_config* out);

/* 1 if `config` can run the given layouts (tile shape compiled, fields in range), else 0. */
int rocm_sgemm_config_supported(const rocm_sgemm_config* config, int layout_c, int layout_a,
                                int layout_b);

/*
 * Workgroup id -> output tile under the XCD-aware order the kernels use (replaces the reference's
 * tile_mapper, kernel/mapping.hpp:211-237).  Host-only; exposed so tests can check it is a
 * bijection of [0, grid_m * grid_n).
 */
int rocm_sgemm_map_workgroup(int workgroup, int grid_m, int grid_n, int group_m, int* tile_m,
                             int* tile_n);

/*
 * Frees the workspace buffers described at the top.  Waits for the current work of the devices
 * concerned; later calls allocate again on demand.  The reference keeps no workspace (its kernels
 * never split K), so this has no counterpart there.
 */
void rocm_sgemm_release_workspaces(void);

/* Message for the last non-OK status returned on the calling thread ("" if none). */
const char* rocm_sgemm_last_error(void);

/* "major.minor.patch (gfx950)". */
const char* rocm_sgemm_version(void);

#ifdef __cplusplus
}
#endif

#endif /* ROCM_SGEMM_C_H */
