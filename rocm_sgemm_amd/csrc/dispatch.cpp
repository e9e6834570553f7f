// Kernel dispatch: the family of compiled kernels, validation of a call, choice of the kernel
// variant, workspace, launches.  Covers what the reference splits over src/gemm.cpp:8-41,
// kernel_launcher.hpp:40-99 and the generated kernel_lookup.cpp (generate_config.py:415-545).

#include "dispatch.hpp"

#include <atomic>
#include <climits>
#include <cmath>
#include <cstdint>
#include <limits>
#include <map>
#include <functional>
#include <mutex>
#include <thread>

#include "launch.hpp"
#include "splitk_reduce.hpp"

namespace rocm_sgemm
{
namespace detail
{

struct tile_shape
{
    int macro_m, macro_n, k_tile, waves_m, waves_n, mfma, stages, waves_k;
};

struct kernel_family_row
{
    tile_shape shape;
    // [X depth-contiguous][Y depth-contiguous][variant]
    //   0: full tiles (direct-to-LDS when stages >= 2)
    //   1: edge-masked, register-staged (stages = 0 shapes; null otherwise)
    //   2: edge-masked direct-to-LDS, 16-byte loads (null for stages = 0 shapes)
    //   3: edge-masked direct-to-LDS, 4-byte loads (null for stages = 0 shapes)
    launch_fn launch[2][2][4];
};

#include "kernel_table.inc"

namespace
{

const kernel_family_row* find_shape(int bm, int bn, int bk, int wm, int wn, int mfma, int stages, int waves_k)
{
    const int wk = waves_k < 1 ? 1 : waves_k; // 0 (a config written before the field existed) = none
    for(int i = 0; i < kernel_family_size; ++i)
    {
        const tile_shape& s = kernel_family[i].shape;
        if(s.macro_m == bm && s.macro_n == bn && s.k_tile == bk && s.waves_m == wm
           && s.waves_n == wn && s.mfma == mfma && s.stages == stages && s.waves_k == wk)
        {
            return &kernel_family[i];
        }
    }
    return nullptr;
}

std::string describe(const rocm_sgemm_config& c)
{
    return "macro " + std::to_string(c.macro_m) + "x" + std::to_string(c.macro_n) + ", k_tile "
           + std::to_string(c.k_tile) + ", waves " + std::to_string(c.waves_m) + "x"
           + std::to_string(c.waves_n) + (c.waves_k > 1 ? "x" + std::to_string(c.waves_k) : std::string())
           + ", mfma " + std::to_string(c.mfma) + ", stages " + std::to_string(c.stages);
}

bool is_layout(int v)
{
    return v == ROCM_SGEMM_ROW_MAJOR || v == ROCM_SGEMM_COL_MAJOR;
}

// Largest dimension the kernels' 32-bit index arithmetic handles (row + tile offsets stay < 2^31).
constexpr size_t max_dim = static_cast<size_t>(INT_MAX) - 4096;

bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// Workspace for split-K / stream-K partials and for the alpha-beta pass.
//
// One buffer per (device, stream), owned by the library, grown on demand and kept until
// release_workspaces() or process exit.  Work on one stream executes in order, so consecutive
// calls on a stream can share a buffer without any synchronisation, and a call costs no
// allocation at all once the buffer is large enough.  (A stream-ordered hipMallocAsync /
// hipFreeAsync pair per call was measured to stall the host until the GPU had caught up, which
// serialises back-to-back calls.)  Calls on different streams get different buffers, so they may
// overlap.
// Locking: the table is guarded by one mutex that is held for the lookup only; every buffer has a
// mutex of its own that a call holds from "got the pointer" until it has enqueued everything that
// uses the buffer.  Growing a buffer frees the old one after waiting for the device, which is only
// safe if no other thread is between those two points on the same buffer; threads on different
// streams never wait for each other.  Table nodes are never erased (release_workspaces() empties
// them in place), so a pointer to a node stays valid for the life of the process.
// A stream that is being captured into a graph NEVER gets the library's buffer: its address would
// be baked into the graph's kernel nodes, and a later growth or release_workspaces() would leave
// every replay reading and writing freed memory.  A captured call always takes a stream-ordered
// allocation instead, which the capture records as allocation / free nodes: the graph owns its
// workspace.
// hipStreamPerThread is one handle value that names a different stream in every host thread, so
// for it the calling thread is part of the key (0 for every other stream).
struct workspace_key
{
    int         device;
    hipStream_t stream;
    size_t      thread;
    bool        operator<(const workspace_key& o) const
    {
        if(device != o.device) return device < o.device;
        if(stream != o.stream) return stream < o.stream;
        return thread < o.thread;
    }
};
struct workspace_buffer
{
    std::mutex in_use; // held by a call from taking `ptr` until its kernels are enqueued
    void*      ptr   = nullptr;
    size_t     bytes = 0;
};
// Every workspace starts with the counters of the launches that sum their partial tiles
// themselves (kernel::gemm_args::counters): always at the same place, zero when the buffer is
// created and left at zero by every launch that uses them.  The partial tiles follow.
constexpr size_t counter_slots = 16384;
constexpr size_t counter_bytes = counter_slots * sizeof(unsigned);
std::mutex                                workspace_table_lock;
std::map<workspace_key, workspace_buffer> workspaces;

// Returns the buffer in *ptr; *stream_ordered is set when the caller must hipFreeAsync it.
// Otherwise `guard` comes back holding the buffer's mutex and must stay so until the caller has
// enqueued everything that uses the buffer.
hipError_t workspace_get(void** ptr, size_t bytes, hipStream_t stream, bool* stream_ordered,
                         std::unique_lock<std::mutex>& guard)
{
    *stream_ordered = false;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if(hipStreamIsCapturing(stream, &capture) != hipSuccess)
    {
        (void)hipGetLastError();
        capture = hipStreamCaptureStatusNone;
    }
    if(capture != hipStreamCaptureStatusNone)
    {
        *stream_ordered = true;
        return hipMallocAsync(ptr, bytes, stream);
    }
    int        device = 0;
    hipError_t err    = hipGetDevice(&device);
    if(err != hipSuccess) return err;
    const size_t thread = stream == hipStreamPerThread ? std::hash<std::thread::id>{}(std::this_thread::get_id()) : 0;
    workspace_buffer* buf;
    {
        std::lock_guard<std::mutex> table(workspace_table_lock);
        buf = &workspaces[workspace_key{device, stream, thread}];
    }
    guard = std::unique_lock<std::mutex>(buf->in_use);
    if(buf->bytes >= bytes)
    {
        *ptr = buf->ptr;
        return hipSuccess;
    }
    // Grow.  The old buffer may still be in use by work queued on this stream; hipFree waits for
    // the device, which is acceptable for an event that happens a handful of times per process.
    if(buf->ptr != nullptr)
    {
        (void)hipFree(buf->ptr);
        buf->ptr   = nullptr;
        buf->bytes = 0;
    }
    const size_t want = bytes + bytes / 4; // head room: slightly larger problems do not regrow
    err               = hipMalloc(&buf->ptr, want);
    if(err == hipSuccess)
    {
        err = hipMemset(buf->ptr, 0, counter_bytes < want ? counter_bytes : want); // the counters start at zero
        if(err != hipSuccess)
        {
            (void)hipFree(buf->ptr);
        }
    }
    if(err != hipSuccess)
    {
        buf->ptr = nullptr;
        return err;
    }
    buf->bytes = want;
    *ptr       = buf->ptr;
    return hipSuccess;
}

// Scratch of the allocation-free entry point: a fixed array in device memory that exists from the
// moment the library's code object is loaded on a GPU until the process ends (each GPU holds its
// own copy at its own address).  On the host the array's name is only a handle for
// hipGetSymbolAddress, not a device address; the address is looked up once per device, with that
// device current, and only that pointer is ever handed to a kernel.
// It is laid out like an allocated workspace: the counters (zero from the start, like all of the
// array), then ROCM_SGEMM_NO_ALLOC_SCRATCH_BYTES for partial tiles.
constexpr size_t scratch_floats = ROCM_SGEMM_NO_ALLOC_SCRATCH_BYTES / sizeof(float);
static __device__ __align__(256) float scratch[counter_bytes / sizeof(float) + scratch_floats];

constexpr int       scratch_max_devices = 64;
std::atomic<float*> scratch_address[scratch_max_devices];

hipError_t scratch_get(float** ptr)
{
    int        device = 0;
    hipError_t err    = hipGetDevice(&device);
    if(err != hipSuccess) return err;
    if(device < 0 || device >= scratch_max_devices) return hipErrorInvalidDevice;
    float* known = scratch_address[device].load(std::memory_order_acquire);
    if(known == nullptr)
    {
        void* found = nullptr;
        err         = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if(err != hipSuccess) return err;
        if(found == nullptr) return hipErrorInvalidSymbol;
        known = static_cast<float*>(found);
        scratch_address[device].store(known, std::memory_order_release); // every thread finds the same value
    }
    *ptr = known;
    return hipSuccess;
}

// CUs of the current device, asked once per process (the library targets one GPU model).
int compute_units()
{
    static const int count = [] {
        int device = 0, n = 0;
        if(hipGetDevice(&device) != hipSuccess
           || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess
           || n < 1)
        {
            n = 256;
        }
        return n;
    }();
    return count;
}

} // namespace

void release_workspaces()
{
    std::lock_guard<std::mutex> table(workspace_table_lock);
    int                         current = -1;
    if(hipGetDevice(&current) != hipSuccess)
    {
        (void)hipGetLastError();
        current = -1;
    }
    for(auto& kv : workspaces)
    {
        std::lock_guard<std::mutex> in_use(kv.second.in_use); // no call is about to enqueue on it
        if(kv.second.ptr != nullptr)
        {
            (void)hipSetDevice(kv.first.device);
            (void)hipFree(kv.second.ptr); // waits for the device: nothing can still be using it
            kv.second.ptr   = nullptr;
            kv.second.bytes = 0;
        }
    }
    if(current >= 0) (void)hipSetDevice(current); // the caller's current device is left as it was
}

int family_size()
{
    return kernel_family_size;
}

void family_entry(int index, rocm_sgemm_config* out)
{
    const tile_shape& s = kernel_family[index].shape;
    *out                = rocm_sgemm_config{s.macro_m, s.macro_n, s.k_tile, s.waves_m, s.waves_n,
                                            s.mfma, s.stages, 1, 4, 0, s.waves_k};
}

bool config_supported(const rocm_sgemm_config& c, int layout_c, int layout_a, int layout_b,
                      std::string& error)
{
    if(!is_layout(layout_a) || !is_layout(layout_b) || !is_layout(layout_c))
    {
        error = "layout must be ROCM_SGEMM_ROW_MAJOR (0) or ROCM_SGEMM_COL_MAJOR (1)";
        return false;
    }
    if(c.split_k < 1 || c.split_k > 1024 || c.group_m < 1 || c.wave_slots < 0 || c.partial_sums < 0
       || c.partial_sums > 2)
    {
        error = "split_k must be in [1, 1024], group_m >= 1, wave_slots >= 0 and partial_sums 0, 1 or 2";
        return false;
    }
    const bool swap = layout_c == ROCM_SGEMM_COL_MAJOR;
    const kernel_family_row* row
        = swap ? find_shape(c.macro_n, c.macro_m, c.k_tile, c.waves_n, c.waves_m, c.mfma, c.stages, c.waves_k)
               : find_shape(c.macro_m, c.macro_n, c.k_tile, c.waves_m, c.waves_n, c.mfma, c.stages, c.waves_k);
    if(row == nullptr)
    {
        error = "No kernel available for the requested configuration and layout (" + describe(c)
                + ")";
        return false;
    }
    return true;
}

int run_gemm(const rocm_sgemm_config& c,
             int                      layout_c,
             int                      layout_a,
             int                      layout_b,
             float*                   C,
             const float*             A,
             const float*             B,
             size_t                   M,
             size_t                   N,
             size_t                   K,
             hipStream_t              stream,
             std::string&             error)
{
    const gemm_problem p{layout_c, layout_a, layout_b, C, A, B, M, N, K, 0, 0, 0, 0, 0, 0, 1, 1.0f, 0.0f};
    return run_gemm(c, p, stream, error);
}

int run_gemm(const rocm_sgemm_config& c, const gemm_problem& p, hipStream_t stream, std::string& error)
{
    const size_t M = p.M, N = p.N, K = p.K;
    if(p.C == nullptr || p.A == nullptr || p.B == nullptr)
    {
        error = "A, B and C must be non-null device pointers";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    if(M == 0 || N == 0 || K == 0)
    {
        error = "matrix dimensions must be positive";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    if(M > max_dim || N > max_dim || K > max_dim)
    {
        error = "matrix dimension exceeds the supported maximum (2^31 - 4097)";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    if(!is_layout(p.layout_a) || !is_layout(p.layout_b) || !is_layout(p.layout_c))
    {
        error = "layout must be ROCM_SGEMM_ROW_MAJOR (0) or ROCM_SGEMM_COL_MAJOR (1)";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    if(c.split_k < 1 || c.split_k > 1024 || c.group_m < 1 || c.wave_slots < 0 || c.partial_sums < 0
       || c.partial_sums > 2)
    {
        error = "split_k must be in [1, 1024], group_m >= 1, wave_slots >= 0 and partial_sums 0, 1 or 2";
        return ROCM_SGEMM_STATUS_BAD_CONFIG;
    }
    if(p.batch < 1 || p.batch > 65535)
    {
        error = "batch count must be in [1, 65535]";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }

    // Leading dimensions: 0 means packed; otherwise at least the contiguous extent.
    const bool   a_row = p.layout_a == ROCM_SGEMM_ROW_MAJOR, b_row = p.layout_b == ROCM_SGEMM_ROW_MAJOR;
    const bool   c_row = p.layout_c == ROCM_SGEMM_ROW_MAJOR;
    const size_t a_min = a_row ? K : M, b_min = b_row ? N : K, c_min = c_row ? N : M;
    const size_t lda = p.lda ? p.lda : a_min, ldb = p.ldb ? p.ldb : b_min, ldc = p.ldc ? p.ldc : c_min;
    if(lda < a_min || ldb < b_min || ldc < c_min || lda > max_dim || ldb > max_dim || ldc > max_dim)
    {
        error = "leading dimension smaller than the matrix extent along its contiguous dimension "
                "(or above 2^31 - 4097)";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    // floats from an operand's origin to one past its last element
    const long long a_extent = static_cast<long long>((a_row ? M : K) - 1) * lda + a_min;
    const long long b_extent = static_cast<long long>((b_row ? K : N) - 1) * ldb + b_min;
    const long long c_extent = static_cast<long long>((c_row ? M : N) - 1) * ldc + c_min;
    if(p.stride_a < 0 || p.stride_b < 0 || p.stride_c < 0)
    {
        error = "batch strides must not be negative";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    if(p.batch > 1 && p.stride_c < c_extent)
    {
        error = "batch stride of C is smaller than one C matrix: the outputs would overlap";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }

    // A column-major C (M x N) is the row-major N x M matrix C^T = B^T * A^T, and a column-major
    // B is a row-major B^T (and so on), so that case runs the same kernels with the operands, the
    // problem shape and the tile shape swapped.
    const bool swap = !c_row;

    kernel::gemm_args args{};
    bool              x_kc, y_kc;
    int               bm, bn, wm, wn;
    if(!swap)
    {
        args.X = p.A, args.Y = p.B;
        args.rows = static_cast<int>(M), args.cols = static_cast<int>(N);
        x_kc = a_row; // A row-major: K contiguous
        y_kc = !b_row; // B column-major: K contiguous
        bm = c.macro_m, bn = c.macro_n, wm = c.waves_m, wn = c.waves_n;
        args.ldx = static_cast<int>(lda), args.ldy = static_cast<int>(ldb);
        args.stride_x = p.stride_a, args.stride_y = p.stride_b;
        args.extent_x = a_extent, args.extent_y = b_extent;
    }
    else
    {
        args.X = p.B, args.Y = p.A;
        args.rows = static_cast<int>(N), args.cols = static_cast<int>(M);
        x_kc = !b_row; // B^T (N x K) row-major
        y_kc = a_row; // A^T (K x M) column-major
        bm = c.macro_n, bn = c.macro_m, wm = c.waves_n, wn = c.waves_m;
        args.ldx = static_cast<int>(ldb), args.ldy = static_cast<int>(lda);
        args.stride_x = p.stride_b, args.stride_y = p.stride_a;
        args.extent_x = b_extent, args.extent_y = a_extent;
    }
    args.P        = p.C;
    args.ldp      = static_cast<int>(ldc);
    args.stride_p = p.stride_c;
    args.depth    = static_cast<int>(K);
    // alpha != 1 or beta != 0: the kernel writes the plain product into a packed workspace and the
    // reduction kernel (a one-slice "sum") blends it into C.  The kernels themselves never scale:
    // touching the accumulators with vector ALU instructions would pull them out of the
    // accumulation registers and cost the 256-accumulator shapes their register budget.
    const bool scaled = !(p.alpha == 1.0f && p.beta == 0.0f);

    const kernel_family_row* row = find_shape(bm, bn, c.k_tile, wm, wn, c.mfma, c.stages, c.waves_k);
    if(row == nullptr)
    {
        error = "No kernel available for the requested configuration and layout (" + describe(c)
                + ")";
        return ROCM_SGEMM_STATUS_NO_KERNEL;
    }
    const int bk = c.k_tile;

    // The kernels address a K-tile with 32-bit byte offsets from its origin: the farthest element
    // of a depth-contiguous tile is (tile rows) * ld floats away, of a row-contiguous one
    // (k_tile) * ld.  Keep that below 2^29 floats (2 GiB).
    {
        const unsigned long long ldx   = static_cast<unsigned long long>(args.ldx);
        const unsigned long long ldy   = static_cast<unsigned long long>(args.ldy);
        const unsigned long long x_far = (x_kc ? bm : bk) * ldx + (x_kc ? bk : bm);
        const unsigned long long y_far = (y_kc ? bn : bk) * ldy + (y_kc ? bk : bn);
        if(x_far >= (1ull << 29) || y_far >= (1ull << 29))
        {
            error = "leading dimension too large for the " + std::to_string(bm) + "x"
                    + std::to_string(bn) + "x" + std::to_string(bk)
                    + " tile (tile extent x leading dimension must stay below 2^29 elements)";
            return ROCM_SGEMM_STATUS_INVALID_ARG;
        }
    }

    args.grid_m  = (args.rows + bm - 1) / bm;
    args.grid_n  = (args.cols + bn - 1) / bn;
    args.group_m = c.group_m;

    // K slices: equal multiples of the K-tile; a slice count that would leave empty slices shrinks.
    const int k_tiles     = (args.depth + bk - 1) / bk;
    int       split       = c.split_k < k_tiles ? c.split_k : k_tiles;
    const int slice_tiles = (k_tiles + split - 1) / split;
    split                 = (k_tiles + slice_tiles - 1) / slice_tiles;
    args.split_k          = split;
    args.k_slice          = split > 1 ? slice_tiles * bk : args.depth;

    // Full tiles of 16-byte aligned lines: the kernel without masks (direct-to-LDS if the shape
    // has one, whose loads fault on a misaligned address).  Anything else: the edge-masked kernel.
    const bool to_workspace  = split > 1 || scaled; // the kernel then writes packed partials only
    // An operand can travel 16 bytes per lane when every line of it starts on a 16-byte boundary
    // (a misaligned load of that size faults) and, if it is stored depth-contiguous, its rows end
    // on one (whole 16-byte pieces beyond K are dropped; one straddling the end of a row could
    // not be).  Only two masked kernels exist per shape: both operands 16 bytes per lane, or both
    // 4 bytes per lane (which needs no alignment), so one operand that cannot go wide takes the
    // other with it.
    const bool x_aligned = aligned16(args.X) && args.ldx % 4 == 0 && (p.batch == 1 || args.stride_x % 4 == 0);
    const bool y_aligned = aligned16(args.Y) && args.ldy % 4 == 0 && (p.batch == 1 || args.stride_y % 4 == 0);
    const bool out_aligned   = to_workspace
                               || (aligned16(p.C) && args.ldp % 4 == 0
                                   && (p.batch == 1 || args.stride_p % 4 == 0));
    const bool full = args.rows % bm == 0 && args.cols % bn == 0 && args.depth % bk == 0 && x_aligned
                      && y_aligned && out_aligned;
    // Full tiles of 16-byte aligned lines: the kernel without masks.  Anything else runs an
    // edge-masked kernel: a direct-to-LDS shape the one with 16-byte loads if both operands allow
    // them, else the one with 4-byte loads; a register-staged shape its own.
    const bool      both_wide = x_aligned && y_aligned && ((!x_kc && !y_kc) || args.depth % 4 == 0);
    const launch_fn masked    = row->launch[x_kc ? 1 : 0][y_kc ? 1 : 0][2];
    const int       variant   = full ? 0 : (masked == nullptr ? 1 : (both_wide ? 2 : 3));
    launch_fn       fn       = row->launch[x_kc ? 1 : 0][y_kc ? 1 : 0][variant];

    // Stream-K tail.  The matrix pipes of the GPU are saturated by W workgroups (one per CU for
    // workgroups of four or more waves; residency beyond that only overlaps tiles on a CU, it does
    // not finish them sooner), so T tiles take ceil(T / W) tile times and a last wave of
    // r = T mod W tiles leaves W - r CUs idle for one of them.  Instead, the K-tiles of those r
    // tiles are laid end to end and dealt out in equal runs to up to W workgroups (a run touches at
    // most two tiles), whose partial tiles a small second kernel sums: the wave then takes r / W
    // of a tile time.  Applies to a single plain product whose config does not already split K,
    // when the wave is at most 85 % full and the time saved is worth the second pass.
    const long long tiles = static_cast<long long>(args.grid_m) * args.grid_n;
    args.tail_begin       = static_cast<int>(tiles <= INT_MAX ? tiles : INT_MAX);
    args.tail_groups      = 0;
    args.tail_per         = 0;
    long long tail_tiles  = 0;
    if(split == 1 && tiles <= INT_MAX && p.batch == 1 && !scaled)
    {
        // the rule works on the caller's tile shape; swapping operands for a column-major C does
        // not change the tile count or the tile area
        long long slots = 0, r = 0;
        if(tail_applies(c, tiles, k_tiles, K, compute_units(), &slots, &r))
        {
            const long long runs = r * k_tiles; // K-tiles of the tail, end to end
            long long       per  = (runs + slots - 1) / slots;
            per                  = per < 4 ? 4 : per; // per <= k_tiles because r <= slots, k_tiles >= 8
            args.tail_per        = static_cast<int>(per);
            args.tail_groups     = static_cast<int>((runs + per - 1) / per);
            args.tail_begin      = static_cast<int>(tiles - r);
            tail_tiles           = r;
        }
    }

    const unsigned long long groups
        = args.tail_groups > 0
              ? static_cast<unsigned long long>(args.tail_begin) + args.tail_groups
              : static_cast<unsigned long long>(tiles) * split;
    if(groups > static_cast<unsigned long long>(INT_MAX))
    {
        error = "problem needs more than 2^31 - 1 workgroups";
        return ROCM_SGEMM_STATUS_INVALID_ARG;
    }
    const unsigned batches = static_cast<unsigned>(p.batch);

    const size_t count = static_cast<size_t>(args.rows) * static_cast<size_t>(args.cols);
    size_t       workspace_floats = 0;
    bool         workspace_stream_ordered = false;
    std::unique_lock<std::mutex> workspace_guard; // held from "got the buffer" to "all enqueued"
    if(split > 1 || scaled)
    {
        workspace_floats = count * split * p.batch;
    }
    else if(args.tail_groups > 0)
    {
        workspace_floats = static_cast<size_t>(args.tail_groups) * 2 * bm * bn;
    }
    // Who adds the partial tiles up: a second kernel, or - only where the config asks for it
    // (partial_sums = 2) - the launch itself: the wave that completes a tile's counter, see
    // kernel::gemm_args::counters.  The second saves a launch and the summing of one tile overlaps
    // with the multiplication of others, but every wave must wait until its write-through stores
    // have been acknowledged before it may draw its ticket, and the wave that adds up reads all
    // parts of its share one after the other.  Measured after that wait went in (it is what makes
    // the scheme correct) and the main loop lost its stalls: the second kernel wins everywhere it
    // was tried - 2560^3 237.5 against 255.1 us, 1024 x 1024 x 16384 (64 x 64 x 64, four waves
    // along K, split 2) 238.4 against 245.0, 1024 x 1024 x 4096 69.5 against 78.1, 768 x 384 x 2304
    // 24.5 against 27.3 - so it is the default (partial_sums = 0 and 1 mean the same); the tuner
    // still times both and records a 2 where the launch wins.
    // (Possible at all only with at most four waves that own at most a 64 x 64 share of the tile
    // each, kernel::tile_config::SUMS_IN_LAUNCH, 32-bit byte offsets into a partial matrix, and
    // counters for every (batch, tile, wave).)
    const int    waves_per_group = wm * wn * (c.waves_k > 1 ? c.waves_k : 1);
    const size_t counters_needed
        = static_cast<size_t>(p.batch) * static_cast<size_t>(args.tail_groups > 0 ? tail_tiles : tiles) * waves_per_group;
    const bool possible = !scaled && (split > 1 || args.tail_groups > 0) && counters_needed <= counter_slots
                          && bm * bn / waves_per_group <= 64 * 64 && waves_per_group <= 4 && count < (1ull << 29);
    bool       in_launch = possible && c.partial_sums == 2;
    if(p.workspace_bytes_out != nullptr)
    {
        *p.workspace_bytes_out = workspace_floats * sizeof(float);
        return ROCM_SGEMM_STATUS_OK;
    }
    void* workspace_base = nullptr;
    if(workspace_floats > 0 && p.no_alloc)
    {
        // the fixed scratch array of this GPU: nothing is allocated, every call on the GPU shares it
        if(workspace_floats > scratch_floats)
        {
            error = "this problem needs " + std::to_string(workspace_floats * sizeof(float))
                    + " bytes of workspace for its partial products; the allocation-free entry point has "
                    + std::to_string(scratch_floats * sizeof(float))
                    + " (use rocm_sgemm_f32, which allocates its workspace)";
            return ROCM_SGEMM_STATUS_WORKSPACE_TOO_LARGE;
        }
        float*     ws  = nullptr;
        hipError_t err = scratch_get(&ws);
        if(err != hipSuccess)
        {
            error = std::string("address of the scratch array not available: ") + hipGetErrorString(err);
            return ROCM_SGEMM_STATUS_LAUNCH_FAILED;
        }
        workspace_base = ws;
    }
    else if(workspace_floats > 0)
    {
        // the library's buffer of this stream (see workspace_get)
        void*      ws  = nullptr;
        hipError_t err = workspace_get(&ws, counter_bytes + workspace_floats * sizeof(float), stream,
                                       &workspace_stream_ordered, workspace_guard);
        if(err != hipSuccess)
        {
            error = std::string("workspace allocation failed: ") + hipGetErrorString(err);
            return ROCM_SGEMM_STATUS_LAUNCH_FAILED;
        }
        workspace_base = ws;
        // a one-off allocation (stream capture) comes with counters that nobody has cleared
        in_launch = in_launch && !workspace_stream_ordered;
    }
    if(workspace_base != nullptr)
    {
        args.partial  = reinterpret_cast<float*>(static_cast<char*>(workspace_base) + counter_bytes);
        args.counters = in_launch ? static_cast<unsigned*>(workspace_base) : nullptr;
    }
    const int       ldc_out    = args.ldp;
    const long long stride_out = args.stride_p;
    if(scaled && split == 1)
    {
        // the workspace stands in for the output: packed, one matrix per batch
        args.P        = args.partial;
        args.ldp      = args.cols;
        args.stride_p = static_cast<long long>(count);
    }

    const kernel::output_scale scale{p.alpha, p.beta};
    hipError_t err = fn(args, static_cast<unsigned>(groups), batches, stream);
    if(args.counters != nullptr)
    {
        // the launch has summed its partial tiles itself
    }
    else if(err == hipSuccess && (split > 1 || scaled))
    {
        const bool vec4 = args.cols % 4 == 0 && ldc_out % 4 == 0 && aligned16(p.C)
                          && (batches == 1 || stride_out % 4 == 0);
        const size_t   want = ((vec4 ? count / 4 : count) + 255) / 256;
        const unsigned grid = static_cast<unsigned>(want < 8192 ? want : 8192);
        if(vec4)
            hipLaunchKernelGGL(kernel::splitk_reduce_vec4_kernel, dim3(grid, batches), dim3(256), 0, stream,
                               p.C, args.partial, args.rows, args.cols, ldc_out, stride_out, split, scale);
        else
            hipLaunchKernelGGL(kernel::splitk_reduce_kernel, dim3(grid, batches), dim3(256), 0, stream,
                               p.C, args.partial, args.rows, args.cols, ldc_out, stride_out, split, scale);
        err = hipPeekAtLastError();
    }
    else if(err == hipSuccess && args.tail_groups > 0)
    {
        const unsigned strips = static_cast<unsigned>((bm * bn / 4 + 255) / 256);
        hipLaunchKernelGGL(kernel::tail_reduce_kernel,
                           dim3(static_cast<unsigned>(tail_tiles), strips < 16 ? strips : 16),
                           dim3(256), 0, stream, p.C, args.partial, args.rows, args.cols, args.ldp,
                           args.grid_m, args.grid_n, args.group_m, args.tail_begin, k_tiles, args.tail_per,
                           bm, bn, scale);
        err = hipPeekAtLastError();
    }
    if(workspace_stream_ordered)
    {
        const hipError_t ferr = hipFreeAsync(workspace_base, stream);
        if(err == hipSuccess)
        {
            err = ferr;
        }
    }
    if(err != hipSuccess)
    {
        error = std::string("kernel launch failed: ") + hipGetErrorString(err);
        return ROCM_SGEMM_STATUS_LAUNCH_FAILED;
    }
    return ROCM_SGEMM_STATUS_OK;
}

} // namespace detail
} // namespace rocm_sgemm
