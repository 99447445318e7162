// Host side of librocm_wmma_gemm_gfx950.so: the templated gemm<> entry points, the
// config lookup, the launch, and the C ABI that the runtime loader binds.
//
// Interface parity: reference rocm_wmma_gemm/src/gemm.cpp:8-53 (dispatch),
// :56-198 (explicit instantiations), :207-250 (C ABI).
#include <rocm_wmma_gemm/gemm.hpp>
#include <rocm_wmma_gemm_c.h>

#include <algorithm>
#include <atomic>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <type_traits>
#include <utility>

#include "config_select.hpp"
#include "kernel_table.hpp"
#include "workspace_policy.hpp"

namespace rocm_wmma_gemm
{
namespace host
{

// LDS per workgroup: the staged pipeline double-buffers one tile pair; the direct
// pipelines keep a ring of 2 (BLOCK_K 64) or 4 (BLOCK_K 32, and pipeline 6) tile pairs.
constexpr int ring_bytes(int bm, int bn, int bk, int pipeline)
{
    if(pipeline == 7)
    {
        // as many stages as fit 76 KB, at least 3 and at most 8 (device::stream_gemm::DEPTH)
        const int stage = (bm + bn) * bk * 2, fit = 76 * 1024 / stage, depth = fit < 3 ? 3 : fit;
        return (depth < 8 ? depth : 8) * stage;
    }
    return (pipeline == 6 || (pipeline != 0 && bk == 32) ? 4 : 2) * (bm + bn) * bk * 2;
}

// (the streaming kernel always runs 4 waves: they split K, not the tile)
constexpr int workgroup_threads(int wm, int wn, int pipeline)
{
    return pipeline == 7 ? 256 : 64 * wm * wn;
}

#define RWG_VARIANT(IDX, BM, BN, BK, WM, WN, PIPE) \
    {BM, BN, BK, WM, WN, PIPE, ring_bytes(BM, BN, BK, PIPE), workgroup_threads(WM, WN, PIPE)},
const variant_desc variant_table[num_variants] = {
#include "variants.def"
};
#undef RWG_VARIANT

// Variants registered at run time (rocm_wmma_gemm_register_variant: kernels the tuner
// compiled into a library of its own): indices num_variants, num_variants + 1, ...  A
// slot is filled completely before registered_count is raised past it, and never changes
// afterwards except for kernels being added to combinations that had none.
constexpr int max_registered = 64;
struct registered_variant
{
    variant_desc           desc;
    std::atomic<kernel_fn> kernels[num_types][2][2][num_modes];
};
registered_variant registered[max_registered];
std::atomic<int>   registered_count{0};
std::mutex         register_mutex;

int variant_total()
{
    return num_variants + registered_count.load(std::memory_order_acquire);
}

// Description of any variant, compiled or registered (index checked by the caller).
const variant_desc& variant_at(int variant)
{
    return variant < num_variants ? variant_table[variant] : registered[variant - num_variants].desc;
}

kernel_fn lookup_kernel(int type_idx, bool a_kmajor, bool b_kmajor, int variant, int mode)
{
    if(type_idx < 0 || type_idx >= num_types || variant < 0 || variant >= variant_total() || mode < 0
       || mode >= num_modes)
    {
        return nullptr;
    }
    if(variant >= num_variants)
    {
        return registered[variant - num_variants].kernels[type_idx][a_kmajor ? 1 : 0][b_kmajor ? 1 : 0][mode].load(
            std::memory_order_acquire);
    }
    const int key = type_idx * 4 + (a_kmajor ? 2 : 0) + (b_kmajor ? 1 : 0);
    switch(key)
    {
#define RWG_CASE(T, AK, BK_) \
    case T * 4 + AK * 2 + BK_: return kernel_slice_##T##_##AK##_##BK_[variant][mode];
        RWG_CASE(0, 0, 0)
        RWG_CASE(0, 0, 1)
        RWG_CASE(0, 1, 0)
        RWG_CASE(0, 1, 1)
        RWG_CASE(1, 0, 0)
        RWG_CASE(1, 0, 1)
        RWG_CASE(1, 1, 0)
        RWG_CASE(1, 1, 1)
        RWG_CASE(2, 0, 0)
        RWG_CASE(2, 0, 1)
        RWG_CASE(2, 1, 0)
        RWG_CASE(2, 1, 1)
        RWG_CASE(3, 0, 0)
        RWG_CASE(3, 0, 1)
        RWG_CASE(3, 1, 0)
        RWG_CASE(3, 1, 1)
#undef RWG_CASE
        default: return nullptr;
    }
}

namespace
{

constexpr size_t in_bytes = 2;

size_t out_bytes(int type_idx)
{
    return (type_idx == 1 || type_idx == 3) ? 4 : 2;
}

// Every kernel of the library is enqueued through this: the launch's own return code is kept
// per host thread, so that the entry points that return a status report what THEIR launches
// did, not an error some earlier call of anybody's left in the runtime's per-thread error
// state (hipPeekAtLastError cannot tell the two apart).
thread_local hipError_t launch_failure = hipSuccess;

template<class... P, class... A, size_t... I>
void enqueue_impl(void (*kernel)(P...), dim3 grid, dim3 block, hipStream_t stream, std::index_sequence<I...>,
                  A&&... a)
{
    std::tuple<std::remove_cv_t<std::remove_reference_t<P>>...> params(std::forward<A>(a)...);
    void*            ptrs[] = {static_cast<void*>(&std::get<I>(params))...};
    const hipError_t rc = hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, 0, stream);
    if(rc != hipSuccess && launch_failure == hipSuccess)
    {
        launch_failure = rc;
    }
}

template<class... P, class... A>
void enqueue(void (*kernel)(P...), dim3 grid, dim3 block, hipStream_t stream, A&&... a)
{
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    enqueue_impl(kernel, grid, block, stream, std::index_sequence_for<P...>{}, std::forward<A>(a)...);
}

// Arrival counters of the whole-K streaming kernel's K slices (one per tile and batch entry
// of a launch).  A counter holds (epoch << 8 | arrivals): the host gives every launch that
// shares tiles an epoch of its own, a workgroup that finds another epoch in its counter
// starts counting from zero, and the workgroup that finishes a tile puts the count back to
// zero, so a replay of a captured launch (same epoch) starts from zero too and a count that
// a killed kernel left behind cannot be mistaken for this launch's.  Two arrays per GPU:
// one for the calls that lease the library's scratch buffer (the lease orders them, so they
// never count in the same slots at the same time), one for the entry point that allocates
// nothing, which takes no lease (its calls are ordered by the caller, like their scratch
// array); a call of one kind never meets a call of the other in a counter.
constexpr size_t stream_arrival_slots = 4096;
__attribute__((used)) static __device__ unsigned int stream_arrivals[stream_arrival_slots];
__attribute__((used)) static __device__ unsigned int noalloc_arrivals[stream_arrival_slots];
std::mutex            arrivals_mutex;
unsigned int*         arrivals_address[64][2] = {};
std::atomic<unsigned> arrival_epoch{0};

unsigned int* arrivals_of_current_device(bool noalloc)
{
    int dev = -1;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    {
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(arrivals_mutex);
    if(arrivals_address[dev][0] == nullptr)
    {
        void *p = nullptr, *q = nullptr;
        if(hipGetSymbolAddress(&p, HIP_SYMBOL(stream_arrivals)) != hipSuccess || p == nullptr
           || hipGetSymbolAddress(&q, HIP_SYMBOL(noalloc_arrivals)) != hipSuccess || q == nullptr)
        {
            (void)hipGetLastError();
            return nullptr;
        }
        arrivals_address[dev][0] = static_cast<unsigned int*>(p);
        arrivals_address[dev][1] = static_cast<unsigned int*>(q);
    }
    return arrivals_address[dev][noalloc ? 1 : 0];
}

// an epoch for one launch that shares tiles: 24 bits, never zero (a fresh counter reads zero)
unsigned int next_arrival_epoch()
{
    unsigned int e;
    do
    {
        e = (arrival_epoch.fetch_add(1, std::memory_order_relaxed) + 1) & 0xffffffu;
    } while(e == 0);
    return e;
}

// Library-owned scratch memory, one buffer per device: fp32 partial planes of split-K
// and zero-padded copies of ragged or misaligned operands.  Allocated on first use,
// grown when a call needs more (after a device-wide synchronisation, since kernels of
// earlier calls may still be reading the old buffer), never shrunk.  What a call may do
// with the buffer is decided by workspace_decide (workspace_policy.hpp).
constexpr size_t workspace_first_bytes = size_t{256} << 20;
constexpr size_t workspace_limit_bytes = size_t{16} << 30;
constexpr int    max_devices           = 64;
std::mutex       workspace_mutex;
char*            workspace_ptr[max_devices]  = {};
size_t           workspace_size[max_devices] = {};
// whether the buffer's address may sit in a captured graph: such a buffer is never freed
bool workspace_lent_to_capture[max_devices] = {};
// The call that used the buffer last: its stream, and an event recorded behind its last
// kernel.
hipStream_t workspace_stream[max_devices]   = {};
hipEvent_t  workspace_released[max_devices] = {};
bool        workspace_used[max_devices]     = {};

// One call's hold on the current device's buffer, from before its first kernel that
// touches the buffer is enqueued until after its last one is.  Calls that need the
// buffer are put in a queue on the device, whatever streams they are on: a call on
// another stream than the previous holder's makes its stream wait (on the device, the
// host never blocks) for the event recorded behind that holder's last kernel, so two
// streams may issue split-K or padded-copy GEMMs at the same time, from one host thread
// or several, as they may with the kernels that need no scratch memory.  A stream under
// graph capture is left out of this: it records and waits for nothing (the caller orders
// the replays of such a graph against other work that uses the buffer), it never
// allocates, frees or synchronises, and a buffer it was given stays allocated for good.
class workspace_lease
{
public:
    workspace_lease() = default;
    workspace_lease(const workspace_lease&)            = delete;
    workspace_lease& operator=(const workspace_lease&) = delete;

    // nullptr: no memory (or too much asked for, or the stream is capturing and the
    // buffer is not there yet or too small); the lease then holds nothing
    char* acquire(size_t bytes, hipStream_t stream)
    {
        if(bytes > workspace_limit_bytes || hipGetDevice(&dev_) != hipSuccess || dev_ < 0
           || dev_ >= max_devices)
        {
            return nullptr;
        }
        hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
        if(hipStreamIsCapturing(stream, &capture) != hipSuccess)
        {
            (void)hipGetLastError();
            capture = hipStreamCaptureStatusNone;
        }
        const bool capturing = capture != hipStreamCaptureStatusNone;
        lock_                = std::unique_lock<std::mutex>(workspace_mutex);
        const workspace_action action = workspace_decide(workspace_size[dev_], bytes, workspace_limit_bytes,
                                                         capturing, workspace_lent_to_capture[dev_]);
        if(action == workspace_action::refuse)
        {
            lock_.unlock();
            return nullptr;
        }
        if(action != workspace_action::use_existing)
        {
            if(action == workspace_action::grow_free_old)
            {
                (void)hipDeviceSynchronize();
                (void)hipFree(workspace_ptr[dev_]);
            }
            // (grow_retire_old: the old buffer stays allocated until the process ends,
            // for the graphs that hold its address)
            workspace_ptr[dev_]             = nullptr;
            workspace_size[dev_]            = 0;
            workspace_used[dev_]            = false;
            workspace_lent_to_capture[dev_] = false;
            const size_t want = workspace_grown_size(bytes, workspace_first_bytes);
            void*        p    = nullptr;
            if(hipMalloc(&p, want) != hipSuccess)
            {
                (void)hipGetLastError();
                lock_.unlock();
                return nullptr;
            }
            workspace_ptr[dev_]  = static_cast<char*>(p);
            workspace_size[dev_] = want;
        }
        stream_  = stream;
        ordered_ = !capturing;
        if(capturing)
        {
            workspace_lent_to_capture[dev_] = true;
        }
        if(ordered_ && workspace_released[dev_] == nullptr
           && hipEventCreateWithFlags(&workspace_released[dev_], hipEventDisableTiming) != hipSuccess)
        {
            (void)hipGetLastError();
            workspace_released[dev_] = nullptr;
            ordered_                 = false;
        }
        if(ordered_ && workspace_used[dev_] && workspace_stream[dev_] != stream)
        {
            (void)hipStreamWaitEvent(stream, workspace_released[dev_], 0);
        }
        held_ = true;
        return workspace_ptr[dev_];
    }

    ~workspace_lease()
    {
        if(held_ && ordered_)
        {
            (void)hipEventRecord(workspace_released[dev_], stream_);
            workspace_stream[dev_] = stream_;
            workspace_used[dev_]   = true;
        }
    }

private:
    std::unique_lock<std::mutex> lock_;
    hipStream_t                  stream_  = nullptr;
    int                          dev_     = 0;
    bool                         held_    = false;
    bool                         ordered_ = false;
};

// Scratch memory that a call brings along instead of leasing the library's buffer (the
// entry point that allocates nothing): the call takes what it needs from the front, or
// fails when it needs more than there is.
struct fixed_scratch
{
    char*  ptr;
    size_t bytes;
};

bool aligned16(const void* p)
{
    return (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
}

// The problem as the kernels see it: C row-major, operands tagged by whether K is
// their contiguous dimension.
struct kernel_problem
{
    void*       C;
    const void* A;
    const void* B;
    size_t      M, N, K, batch;
    bool        a_kmajor, b_kmajor;
    size_t      stride_a, stride_b, stride_c;
};

kernel_problem to_kernel_space(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                               size_t batch, int layout_c, int layout_a, int layout_b)
{
    kernel_problem p;
    p.K     = K;
    p.batch = batch;
    p.C     = C;
    if(layout_c == 0)
    {
        p.A        = A;
        p.B        = B;
        p.M        = M;
        p.N        = N;
        p.a_kmajor = layout_a == 0; // row-major M x K: K contiguous
        p.b_kmajor = layout_b == 1; // column-major K x N: K contiguous
        p.stride_a = M * K;
        p.stride_b = K * N;
    }
    else
    {
        // Column-major C (M x N) is the row-major N x M matrix C^T = B^T * A^T.  B^T
        // (N x K) is the same buffer as B with the opposite layout tag, likewise A^T.
        p.A        = B;
        p.B        = A;
        p.M        = N;
        p.N        = M;
        p.a_kmajor = layout_b == 1; // B^T is K-contiguous iff B is column-major
        p.b_kmajor = layout_a == 0; // A^T (K x M) is K-contiguous iff A is row-major
        p.stride_a = K * N;
        p.stride_b = M * K;
    }
    p.stride_c = M * N;
    return p;
}

// CUs of the current device (cached per device), 0 if unknown.
size_t compute_units_of_current_device()
{
    static std::atomic<int> cached[64];
    int dev = 0;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    {
        return 0;
    }
    int cus = cached[dev].load(std::memory_order_relaxed);
    if(cus == 0)
    {
        if(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess)
        {
            return 0;
        }
        cached[dev].store(cus, std::memory_order_relaxed);
    }
    return static_cast<size_t>(cus);
}

int pick_mode(const kernel_problem& p, const variant_desc& v, int split_k)
{
    const bool batch_ok = p.batch == 1 || ((p.stride_a % 8 == 0) && (p.stride_b % 8 == 0));
    const bool a_vec    = (p.a_kmajor ? p.K % 8 == 0 : p.M % 8 == 0) && aligned16(p.A);
    const bool b_vec    = (p.b_kmajor ? p.K % 8 == 0 : p.N % 8 == 0) && aligned16(p.B);
    if(!(a_vec && b_vec && batch_ok))
    {
        return static_cast<int>(device::load_mode::scalar);
    }
    (void)split_k;
    const bool full = p.M % v.block_m == 0 && p.N % v.block_n == 0 && p.K % v.block_k == 0;
    return static_cast<int>(full ? device::load_mode::vec_unguarded
                                 : device::load_mode::vec_guarded);
}

template<class OutT>
void zero_fill(void* C, size_t count, hipStream_t stream)
{
    const int blocks = static_cast<int>(std::min<size_t>((count + 255) / 256, 65535));
    enqueue(&device::fill_zero<OutT>, dim3(blocks), dim3(256), stream, static_cast<OutT*>(C),
            static_cast<long long>(count));
}

// Variant that serves shapes a direct-to-LDS variant cannot take: the staged
// variant with the same workgroup tile, else the small general tile.
int staged_fallback(const variant_desc& v)
{
    for(int i = 0; i < num_variants; ++i)
    {
        const variant_desc& w = variant_table[i];
        if(w.pipeline == 0 && w.block_m == v.block_m && w.block_n == v.block_n)
        {
            return i;
        }
    }
    return 0;
}

// A direct-to-LDS variant other than the persistent kernel with the same workgroup tile
// (the 16x16x32 ping-pong kernel first), else what staged_fallback gives.
int elementwise_store_variant(const variant_desc& v)
{
    for(int pipeline : {4, 2, 3, 1})
    {
        for(int i = 0; i < num_variants; ++i)
        {
            const variant_desc& w = variant_table[i];
            if(w.pipeline == pipeline && w.block_m == v.block_m && w.block_n == v.block_n)
            {
                return i;
            }
        }
    }
    return staged_fallback(v);
}

size_t round_up(size_t x, size_t to)
{
    return (x + to - 1) / to * to;
}

// The direct pipelines address a tile with 32-bit byte offsets from its origin.
bool spans_fit(const variant_desc& v, bool a_kmajor, bool b_kmajor, size_t lda, size_t ldb, int bits = 32)
{
    const unsigned long long a_span = (a_kmajor ? v.block_m : v.block_k) * lda * 2ull;
    const unsigned long long b_span = (b_kmajor ? v.block_n : v.block_k) * ldb * 2ull;
    return a_span < (1ull << bits) && b_span < (1ull << bits);
}

// What the whole-K streaming kernel (pipeline 7) takes: an operand that is not K-contiguous
// with 16-byte aligned k rows; at least one stage of 128 of K (the last
// may be cut short); 16-byte aligned rows, and a stage of a tile within reach of a 31-bit offset.
bool streaming_ok(const kernel_problem& p, const variant_desc& v)
{
    if(!(p.K >= 128 && ((!p.a_kmajor && !p.b_kmajor) || p.K % 8 == 0) && aligned16(p.A) && aligned16(p.B)
         && (p.batch == 1 || (p.stride_a % 8 == 0 && p.stride_b % 8 == 0))))
    {
        return false;
    }
    if((!p.a_kmajor && p.M % 8 != 0) || (!p.b_kmajor && p.N % 8 != 0))
    {
        return false;
    }
    // byte offsets inside a tile: its rows of K elements, or K rows of the operand's width
    const unsigned long long span_a = p.a_kmajor ? 1ull * v.block_m * p.K * 2 : 1ull * p.K * p.M * 2;
    const unsigned long long span_b = p.b_kmajor ? 1ull * v.block_n * p.K * 2 : 1ull * p.K * p.N * 2;
    return span_a < (1ull << 31) && span_b < (1ull << 31);
}

// from this size on the streaming kernel reads an operand with the non-temporal hint (the
// memory-side cache holds 256 MB), and the persistent kernel one that a single row (column) of
// its tiles reads
constexpr size_t stream_once_bytes   = size_t{256} << 20;
constexpr size_t read_once_tile_rows = 1;

template<class OutT>
int launch_streaming(int type_idx, const launch_plan& plan, const kernel_problem& p, hipStream_t stream,
                     const fixed_scratch* fixed)
{
    const variant_desc& v = variant_at(plan.variant);
    if(!streaming_ok(p, v))
    {
        return -1;
    }
    kernel_fn fn = lookup_kernel(type_idx, p.a_kmajor, p.b_kmajor, plan.variant,
                                 static_cast<int>(device::load_mode::vec_guarded));
    if(fn == nullptr)
    {
        return -1;
    }
    const size_t grid_m = (p.M + v.block_m - 1) / v.block_m, grid_n = (p.N + v.block_n - 1) / v.block_n;
    if(grid_m * grid_n > 0x7fffffffull)
    {
        throw std::runtime_error("rocm_wmma_gemm: tile grid too large");
    }
    // plan.split_k = s > 1: s workgroups per tile, each with K / s, added up inside the
    // launch by the last of them to finish.  Needs whole stages per slice, a counter per
    // tile and batch entry, and room for the partial tiles; without them the tiles stay
    // whole.
    const size_t tiles       = grid_m * grid_n;
    const size_t nb_max      = std::min<size_t>(65535, p.batch);
    size_t       slices      = plan.split_k > 1 ? static_cast<size_t>(plan.split_k) : 1;
    const size_t stages      = (p.K + 127) / 128;
    const size_t tile_floats = static_cast<size_t>(v.block_m) * v.block_n;
    if(slices > 1 && (slices > 8 /* device::stream_gemm::MAX_SLICES */ || stages % slices != 0 || tiles * nb_max > stream_arrival_slots || tiles * slices > 0x7fffffffull))
    {
        slices = 1;
    }
    char*           partials = nullptr;
    unsigned int*   arrivals = nullptr;
    workspace_lease lease; // held until the kernel is enqueued
    if(slices > 1)
    {
        const size_t bytes = tiles * nb_max * slices * tile_floats * sizeof(float);
        arrivals           = arrivals_of_current_device(fixed != nullptr);
        if(fixed != nullptr)
        {
            partials = bytes <= fixed->bytes ? fixed->ptr : nullptr;
        }
        else
        {
            partials = lease.acquire(bytes, stream);
        }
        if(partials == nullptr || arrivals == nullptr)
        {
            slices = 1;
        }
    }
    for(size_t b0 = 0; b0 < p.batch; b0 += 65535)
    {
        const size_t      nb = std::min<size_t>(65535, p.batch - b0);
        device::gemm_args args{};
        args.C              = static_cast<char*>(p.C) + b0 * p.stride_c * sizeof(OutT);
        args.A              = static_cast<const char*>(p.A) + b0 * p.stride_a * in_bytes;
        args.B              = static_cast<const char*>(p.B) + b0 * p.stride_b * in_bytes;
        args.M              = static_cast<int>(p.M);
        args.N              = static_cast<int>(p.N);
        args.K              = static_cast<int>(p.K);
        args.lda            = static_cast<long long>(p.a_kmajor ? p.K : p.M);
        args.ldb            = static_cast<long long>(p.b_kmajor ? p.K : p.N);
        args.batch_stride_a = static_cast<long long>(p.stride_a);
        args.batch_stride_b = static_cast<long long>(p.stride_b);
        args.batch_stride_c = static_cast<long long>(p.stride_c);
        args.grid_m         = static_cast<int>(grid_m);
        args.grid_n         = static_cast<int>(grid_n);
        args.group          = 1;
        args.k_slices       = static_cast<int>(slices);
        args.partials       = reinterpret_cast<float*>(partials);
        args.arrivals       = arrivals;
        args.arrival_epoch  = slices > 1 ? next_arrival_epoch() : 0;
        // an operand that one row (column) of tiles reads once and that cannot stay in the
        // memory-side cache for the next call either is loaded with the non-temporal hint
        args.stream_once    = (grid_m == 1 && p.N * p.K * in_bytes * nb >= stream_once_bytes ? 1 : 0)
                           | (grid_n == 1 && p.M * p.K * in_bytes * nb >= stream_once_bytes ? 2 : 0);
        args.blocks_per_batch = static_cast<int>(tiles);
        args.batches          = static_cast<int>(nb);
        enqueue(fn, dim3(static_cast<unsigned>(tiles * slices), static_cast<unsigned>(nb)), dim3(v.threads), stream,
                args);
    }
    return 0;
}

template<class OutT>
int launch(int type_idx, const launch_plan& plan_in, const kernel_problem& p, hipStream_t stream,
           const fixed_scratch* fixed)
{
    launch_plan plan = plan_in;
    if(plan.variant < 0 || plan.variant >= variant_total())
    {
        return -1;
    }
    if(p.M > 0x7fffffffull || p.N > 0x7fffffffull || p.K > 0x7fffffffull)
    {
        throw std::runtime_error("rocm_wmma_gemm: M, N and K must each fit in 31 bits");
    }

    if(variant_at(plan.variant).pipeline == 7)
    {
        return launch_streaming<OutT>(type_idx, plan, p, stream, fixed);
    }

    // Operand views the kernel will see; may be replaced by padded copies below.
    const void* a_ptr    = p.A;
    const void* b_ptr    = p.B;
    size_t      lda      = p.a_kmajor ? p.K : p.M;
    size_t      ldb      = p.b_kmajor ? p.K : p.N;
    size_t      k_kernel = p.K;
    size_t      stride_a = p.stride_a, stride_b = p.stride_b;
    if(variant_at(plan.variant).pipeline == 5)
    {
        // The persistent kernel stores C in 16-byte pieces through a buffer descriptor per
        // tile: every row of C must start on 16 bytes and hold whole pieces, and a tile's
        // rows must span less than 2 GiB.  Anything else goes to a kernel with the same
        // tile that stores element by element.
        const bool c_pieces = aligned16(p.C) && p.N % 8 == 0 && (p.batch == 1 || p.stride_c % 8 == 0)
                              && p.N < (size_t{1} << 21);
        if(!c_pieces)
        {
            plan.variant = elementwise_store_variant(variant_at(plan.variant));
            if(plan.split_k == -1)
            {
                plan.split_k = 1;
            }
        }
    }
    int         mode     = pick_mode(p, variant_at(plan.variant), plan.split_k);
    size_t      pack_bytes = 0;
    bool        packed     = false; // the kernel reads a padded copy of ...
    bool        copy_a = false, copy_b = false; // ... this operand
    int         k_tail = 0; // columns of a partial last K tile that the kernel cuts off itself

    if(variant_at(plan.variant).pipeline != 0)
    {
        const variant_desc& dv = variant_at(plan.variant);
        const bool direct_ok = mode == static_cast<int>(device::load_mode::vec_unguarded)
                               && spans_fit(dv, p.a_kmajor, p.b_kmajor, lda, ldb);
        if(direct_ok)
        {
            // The 16x16x32 kernels store 4 elements of C at a time when unguarded.
            const bool c_vec = aligned16(p.C) && (p.batch == 1 || p.stride_c % 8 == 0);
            if((dv.pipeline == 3 || dv.pipeline == 4) && !c_vec)
            {
                mode = static_cast<int>(device::load_mode::vec_guarded);
            }
        }
        else if(dv.pipeline == 5 && mode == static_cast<int>(device::load_mode::vec_guarded)
                && spans_fit(dv, p.a_kmajor, p.b_kmajor, lda, ldb, 31))
        {
            // Ragged M, N or K, rows aligned: the persistent kernel takes the operands as
            // they are.  Its buffer descriptors end at the operands' ends, tiles that hang
            // over an edge in M or N read zeros or neighbouring data there, and the guarded
            // stores leave those rows and columns out; of a last K tile that the operands
            // hold only in part the kernel reads the rest as zeros.
            k_kernel = round_up(p.K, dv.block_k);
            k_tail   = static_cast<int>(p.K % dv.block_k);
        }
        else
        {
            // Ragged or misaligned: run the direct kernel on zero-padded copies when the
            // problem is big enough to pay for the copy, else take the staged kernel.  Only
            // an operand that needs it is copied: one whose rows are aligned and whose
            // extents are whole tiles stays where it is (a skinny GEMM pads its small
            // operand and streams the big one from where it lies).
            const size_t m_pad = round_up(p.M, dv.block_m), n_pad = round_up(p.N, dv.block_n),
                         k_pad = round_up(p.K, dv.block_k);
            const bool   strides_ok = p.batch == 1 || (p.stride_a % 8 == 0 && p.stride_b % 8 == 0);
            copy_a = !(k_pad == p.K && m_pad == p.M && strides_ok && aligned16(p.A)
                       && (p.a_kmajor ? p.K : p.M) % 8 == 0);
            copy_b = !(k_pad == p.K && n_pad == p.N && strides_ok && aligned16(p.B)
                       && (p.b_kmajor ? p.K : p.N) % 8 == 0);
            const size_t pa = m_pad * k_pad, pb = k_pad * n_pad;
            const size_t plda = !copy_a ? lda : p.a_kmajor ? k_pad : m_pad;
            const size_t pldb = !copy_b ? ldb : p.b_kmajor ? k_pad : n_pad;
            const size_t copied = (copy_a ? pa : 0) + (copy_b ? pb : 0);
            pack_bytes = round_up(copied * p.batch * in_bytes, 256);
            // padding pays when the GEMM is large next to the copy, which moves every copied
            // element twice: at least 256 FLOP per copied element
            const bool pays = copied > 0 && p.K >= 128
                              && 2.0 * p.M * p.N * p.K / static_cast<double>(copied) >= 256.0;
            if(pays && spans_fit(dv, p.a_kmajor, p.b_kmajor, plda, pldb) && pack_bytes <= workspace_limit_bytes / 2)
            {
                packed   = true;
                lda      = plda;
                ldb      = pldb;
                k_kernel = k_pad;
                stride_a = copy_a ? pa : p.stride_a;
                stride_b = copy_b ? pb : p.stride_b;
                mode     = static_cast<int>(device::load_mode::vec_guarded); // guarded C stores
            }
            else
            {
                pack_bytes   = 0;
                plan.variant = staged_fallback(dv);
                mode         = pick_mode(p, variant_at(plan.variant), plan.split_k);
                if(mode == static_cast<int>(device::load_mode::scalar))
                {
                    // The 2-byte-load path keeps far more values in flight per thread;
                    // the small tile is the variant built to hold them without spilling.
                    plan.variant = 0;
                }
            }
        }
    }
    const variant_desc& v = variant_at(plan.variant);

    const size_t grid_m = (p.M + v.block_m - 1) / v.block_m;
    const size_t grid_n = (p.N + v.block_n - 1) / v.block_n;
    if(grid_m * grid_n > 0x7fffffffull)
    {
        throw std::runtime_error("rocm_wmma_gemm: tile grid too large");
    }

    // plan.split_k > 1: every tile is split (few tiles, long K).  plan.split_k < -1: only
    // the tiles of the last, partial wave over the CUs are split, -split_k ways, so that
    // their workgroups fill the machine too (tiles that do not divide by the CU count
    // otherwise leave most CUs idle for a whole tile time at the end).
    const int k_steps     = static_cast<int>((k_kernel + v.block_k - 1) / v.block_k);
    const size_t tiles    = grid_m * grid_n;
    size_t    tail_begin  = 0; // first split tile
    int       split_k     = 1;
    if(plan.split_k > 1)
    {
        split_k = plan.split_k;
    }
    else if(plan.split_k < -1)
    {
        const size_t cus = compute_units_of_current_device();
        if(cus > 0 && tiles > cus && tiles % cus != 0)
        {
            tail_begin = tiles / cus * cus;
            split_k    = -plan.split_k;
        }
    }
    // Slices hold ceil(k_steps / split_k) K steps each; keep only as many as are not
    // empty (5 steps 4 ways is 2, 2, 1 and nothing for a fourth slice).
    auto without_empty_slices = [k_steps](int slices) {
        if(slices > k_steps)
        {
            slices = k_steps;
        }
        if(slices > 1)
        {
            const int per = (k_steps + slices - 1) / slices;
            slices        = (k_steps + per - 1) / per;
        }
        return slices;
    };
    split_k = without_empty_slices(split_k);
    const size_t split_tiles = tiles - tail_begin;
    if(tail_begin + split_tiles * static_cast<size_t>(split_k) > 0x7fffffffull)
    {
        split_k = 1;
    }
    // fp32 partial sums of one batch entry: whole planes when every tile is split, else
    // one block_m x block_n tile per split tile and slice
    const size_t plane_bytes = tail_begin == 0
                                   ? p.M * p.N * sizeof(float)
                                   : split_tiles * v.block_m * v.block_n * sizeof(float);
    // Batches per launch: bounded by grid.y and, under split-K, by a 1 GiB budget for
    // the partial sums.
    size_t batches_per_launch = std::min<size_t>(p.batch, 65535);
    while(split_k > 1 && plane_bytes * split_k > (size_t{1} << 30))
    {
        split_k = without_empty_slices(split_k - 1);
    }
    if(split_k == 1)
    {
        tail_begin = 0;
    }
    if(split_k > 1)
    {
        batches_per_launch
            = std::min(batches_per_launch, std::max<size_t>((size_t{1} << 30) / (plane_bytes * split_k), 1));
    }
    // A persistent kernel numbers its work items over the whole launch with an int.
    size_t     blocks_per_batch = tail_begin + split_tiles * static_cast<size_t>(split_k);
    const bool persistent       = v.pipeline == 5;
    if(persistent)
    {
        batches_per_launch = std::min(batches_per_launch, std::max<size_t>(0x7fffffffull / blocks_per_batch, 1));
    }
    // plan.split_k == -1, persistent kernel: the workgroups walk by K tile instead of by
    // tile, each over the same number of K tiles of the sequence of all K tiles of the
    // launch; tiles cut by the borders of those ranges are added up from two fp32 slots
    // per workgroup.  For tile counts that fill the CUs badly (144 or 320 tiles on 256).
    size_t stream_groups = 0, stream_units = 0;
    if(persistent && plan.split_k == -1)
    {
        const size_t cus         = compute_units_of_current_device();
        const size_t total_units = tiles * p.batch * static_cast<size_t>(k_steps);
        const size_t chunks      = v.block_m * v.block_n / device::reduce_chunk_elems;
        if(cus > 0 && total_units > 0 && total_units <= 0x7fffffffull && tiles * p.batch * chunks <= 0x7fffffffull)
        {
            stream_groups      = std::min(cus, total_units);
            stream_units       = (total_units + stream_groups - 1) / stream_groups;
            stream_groups      = (total_units + stream_units - 1) / stream_units;
            batches_per_launch = p.batch;
        }
    }
    const size_t partial_bytes = stream_groups > 0
                                     ? 2 * stream_groups * v.block_m * v.block_n * sizeof(float)
                                     : (split_k > 1 ? plane_bytes * split_k * batches_per_launch : 0);

    char*           workspace = nullptr;
    workspace_lease lease; // held until the last kernel of this call is enqueued
    if(pack_bytes + partial_bytes > 0 && fixed != nullptr)
    {
        if(pack_bytes + partial_bytes > fixed->bytes)
        {
            return ROCM_WMMA_GEMM_ERR_SCRATCH;
        }
        workspace = fixed->ptr;
    }
    else if(pack_bytes + partial_bytes > 0)
    {
        workspace = lease.acquire(pack_bytes + partial_bytes, stream);
        if(workspace == nullptr)
        {
            if(packed)
            {
                // no memory for the padded copies: take the general kernel instead
                launch_plan retry = plan;
                retry.variant     = staged_fallback(v);
                if(pick_mode(p, variant_at(retry.variant), retry.split_k)
                   == static_cast<int>(device::load_mode::scalar))
                {
                    retry.variant = 0;
                }
                return launch<OutT>(type_idx, retry, p, stream, fixed);
            }
            split_k          = 1;
            tail_begin       = 0;
            blocks_per_batch = tiles;
            stream_groups    = 0;
            stream_units     = 0;
            if(persistent)
            {
                batches_per_launch = std::min<size_t>(p.batch, std::max<size_t>(0x7fffffffull / tiles, 1));
            }
        }
    }
    float* partials = split_k > 1 || stream_groups > 0 ? reinterpret_cast<float*>(workspace + pack_bytes) : nullptr;

    if(packed)
    {
        auto* wa = reinterpret_cast<unsigned short*>(workspace);
        auto* wb = wa + (copy_a ? stride_a * p.batch : 0);
        // operand as a 2-D array: `outer` rows of `inner` contiguous elements
        const size_t a_outer = p.a_kmajor ? p.M : p.K, a_inner = p.a_kmajor ? p.K : p.M;
        const size_t b_outer = p.b_kmajor ? p.N : p.K, b_inner = p.b_kmajor ? p.K : p.N;
        const size_t a_outer_pad = stride_a / lda, b_outer_pad = stride_b / ldb;
        for(size_t b0 = 0; b0 < p.batch; b0 += 65535)
        {
            const unsigned nb = static_cast<unsigned>(std::min<size_t>(65535, p.batch - b0));
            device::pack_job jobs[2];
            unsigned         count = 0, blocks = 0;
            auto add = [&](const void* src, unsigned short* dst, size_t outer, size_t inner, size_t outer_pad,
                           size_t inner_pad, size_t src_stride, size_t dst_stride) {
                jobs[count++] = {static_cast<const unsigned short*>(src) + b0 * src_stride,
                                 dst + b0 * dst_stride,
                                 static_cast<int>(outer),
                                 static_cast<int>(inner),
                                 static_cast<int>(outer_pad),
                                 static_cast<int>(inner_pad),
                                 static_cast<long long>(src_stride),
                                 static_cast<long long>(dst_stride)};
                blocks = std::max(blocks,
                                  static_cast<unsigned>(std::min<size_t>((outer_pad * (inner_pad / 8) + 255) / 256, 8192)));
            };
            if(copy_a)
            {
                add(p.A, wa, a_outer, a_inner, a_outer_pad, lda, p.stride_a, stride_a);
            }
            if(copy_b)
            {
                add(p.B, wb, b_outer, b_inner, b_outer_pad, ldb, p.stride_b, stride_b);
            }
            if(count == 1)
            {
                jobs[1] = jobs[0];
            }
            // one launch for both operands: a dependent launch costs as much as a small copy
            enqueue(&device::pack_padded<unsigned short>, dim3(blocks, count, nb), dim3(256), stream, jobs[0], jobs[1]);
        }
        if(copy_a)
        {
            a_ptr = wa;
        }
        if(copy_b)
        {
            b_ptr = wb;
        }
    }

    kernel_fn fn = lookup_kernel(type_idx, p.a_kmajor, p.b_kmajor, plan.variant, mode);
    if(fn == nullptr)
    {
        // reference kernel_launcher.hpp:119-125 throws the same way
        throw std::runtime_error("No kernel available for the requested configuration and layout");
    }
    // a plan that walks K in runs takes the kernel's twin built for that, where there is one;
    // so does a problem with an operand of 256 MB and more that one row (column) of tiles
    // reads: the twin with non-temporal loads of that operand (solo_gemm says why)
    int k_run = v.pipeline == 5 ? plan_k_run(plan.touch) : 0;
    int k_group = v.pipeline == 5 ? plan_k_group(plan.touch) : 0;
    const size_t per_launch = std::min(batches_per_launch, p.batch);
    const int    once       = v.pipeline != 5 ? 0
                              : grid_m <= read_once_tile_rows && p.N * p.K * in_bytes * per_launch >= stream_once_bytes ? 1
                              : grid_n <= read_once_tile_rows && p.M * p.K * in_bytes * per_launch >= stream_once_bytes ? 2
                                                                                                                      : 0;
    if(k_run > 0 || k_group > 0 || once != 0)
    {
        auto twin_of = [&](int which) {
            return mode < k_runs_twin - 1 ? lookup_kernel(type_idx, p.a_kmajor, p.b_kmajor, plan.variant,
                                                          mode + k_runs_twin + once_stride * which)
                                          : nullptr;
        };
        kernel_fn twin = twin_of(once);
        if(twin == nullptr && once != 0 && (k_run > 0 || k_group > 0))
        {
            twin = twin_of(0); // (a registered variant may hold the first twins only)
        }
        if(twin != nullptr)
        {
            fn = twin;
        }
        else
        {
            k_run   = 0;
            k_group = 0;
        }
    }

    for(size_t b0 = 0; b0 < p.batch; b0 += batches_per_launch)
    {
        const size_t nb = std::min(batches_per_launch, p.batch - b0);
        device::gemm_args args{};
        args.C = static_cast<char*>(p.C) + b0 * p.stride_c * sizeof(OutT);
        args.A = static_cast<const char*>(a_ptr) + b0 * stride_a * in_bytes;
        args.B = static_cast<const char*>(b_ptr) + b0 * stride_b * in_bytes;
        args.M = static_cast<int>(p.M);
        args.N = static_cast<int>(p.N);
        args.K = static_cast<int>(k_kernel);
        args.lda = static_cast<long long>(lda);
        args.ldb = static_cast<long long>(ldb);
        args.batch_stride_a = static_cast<long long>(stride_a);
        args.batch_stride_b = static_cast<long long>(stride_b);
        args.batch_stride_c = static_cast<long long>(p.stride_c);
        args.grid_m         = static_cast<int>(grid_m);
        args.grid_n         = static_cast<int>(grid_n);
        args.group          = plan.swizzle == 0 ? 1 : plan.swizzle; // negative: bands of tile columns
        args.k_slices       = split_k;
        args.tail_begin     = static_cast<int>(tail_begin);
        args.partials       = partials;
        args.blocks_per_batch = static_cast<int>(blocks_per_batch);
        args.batches          = static_cast<int>(nb);
        args.stream_units     = static_cast<int>(stream_units);
        args.k_tail           = k_tail;
        args.warm_ahead       = persistent ? std::min(plan_touch_distance(plan.touch), 3) : 0;
        args.k_block          = k_run;
        args.k_group          = k_group;


        args.batch_by_xcd     = (persistent || v.pipeline == 6) && nb > 1 && split_k == 1 && stream_groups == 0
                                        && blocks_per_batch * nb < (size_t{1} << 31)
                                    ? 1
                                    : 0;

        dim3 grid(static_cast<unsigned>(blocks_per_batch), static_cast<unsigned>(nb));
        if(persistent)
        {
            // one workgroup per CU (each takes a whole CU), striding over the work items
            const size_t cus   = compute_units_of_current_device();
            const size_t items = blocks_per_batch * nb;
            grid               = dim3(static_cast<unsigned>(cus > 0 ? std::min(items, cus) : items), 1);
            if(stream_groups > 0)
            {
                grid = dim3(static_cast<unsigned>(stream_groups), 1);
            }
        }
        enqueue(fn, grid, dim3(v.threads), stream, args);
        if(stream_groups > 0)
        {
            if(stream_units % static_cast<size_t>(k_steps) != 0)
            {
                // (ranges of whole tiles cut nothing)
                enqueue(&device::reduce_stream_tiles<OutT>,
                        dim3(static_cast<unsigned>(tiles * nb * (v.block_m * v.block_n / device::reduce_chunk_elems))),
                        dim3(256), stream, static_cast<OutT*>(args.C), partials, args.M, args.N, v.block_m,
                        v.block_n, args.grid_m, args.grid_n, args.group, k_steps, args.stream_units,
                        args.batch_stride_c);
            }
            continue;
        }
        if(split_k > 1 && tail_begin == 0)
        {
            const long long plane  = static_cast<long long>(p.M) * static_cast<long long>(p.N);
            const int       blocks = static_cast<int>(std::min<long long>((plane + 255) / 256, 4096));
            enqueue(&device::reduce_partials<OutT>, dim3(blocks, static_cast<unsigned>(nb)), dim3(256), stream,
                    static_cast<OutT*>(args.C), partials, plane, split_k, args.batch_stride_c);
        }
        else if(split_k > 1)
        {
            enqueue(&device::reduce_split_tiles<OutT>,
                    dim3(static_cast<unsigned>((tiles - tail_begin)
                                               * (v.block_m * v.block_n / device::reduce_chunk_elems)),
                         static_cast<unsigned>(nb)),
                    dim3(256), stream, static_cast<OutT*>(args.C), partials, args.M, args.N, v.block_m, v.block_n,
                    args.grid_m, args.grid_n, args.group, args.tail_begin, split_k, args.batch_stride_c);
        }
    }
    return 0;
}

template<class OutT>
int run(int type_idx, const launch_plan* forced, void* C, void* A, void* B, size_t M, size_t N,
        size_t K, size_t batch, int layout_c, int layout_a, int layout_b, hipStream_t stream,
        const fixed_scratch* fixed)
{
    if((layout_c | layout_a | layout_b) & ~1)
    {
        return -2; // reference src/gemm.cpp:243: unknown layout key -> nothing happens
    }
    if(M == 0 || N == 0 || batch == 0)
    {
        return 0;
    }
    if(K == 0)
    {
        zero_fill<OutT>(C, M * N * batch, stream);
        return 0;
    }
    const kernel_problem p = to_kernel_space(C, A, B, M, N, K, batch, layout_c, layout_a, layout_b);
    launch_plan          plan
        = forced ? *forced
                 : select_plan(M, N, K, type_idx, layout_c, layout_a, layout_b, batch,
                               compute_units_of_current_device());
    if(!forced && variant_at(plan.variant).pipeline == 7 && !streaming_ok(p, variant_at(plan.variant)))
    {
        // the dispatcher prices shapes, not pointers: operands that the streaming kernel
        // cannot take (base pointers or batch strides that are not 16-byte aligned) go
        // to the general kernel with the shape heuristic's split
        plan = heuristic_plan(M, N, K, layout_c);
    }
    if(variant_at(plan.variant).pipeline != 0
       && lookup_kernel(type_idx, p.a_kmajor, p.b_kmajor, plan.variant,
                        static_cast<int>(device::load_mode::vec_unguarded))
              == nullptr)
    {
        // a tile that is not built for this pair of operand layouts (tile extents that
        // are no multiple of 128 need that operand K-contiguous)
        if(forced)
        {
            return -1;
        }
        plan.variant = staged_fallback(variant_at(plan.variant));
    }
    if(!forced && variant_at(plan.variant).pipeline == 0)
    {
        // Same rule as in launch() for a staged variant picked directly: misaligned
        // operands go through the small tile.  A direct variant is left alone here:
        // launch() decides between padded copies and the staged kernels.
        const int mode = pick_mode(p, variant_at(plan.variant), plan.split_k);
        if(mode == static_cast<int>(device::load_mode::scalar))
        {
            plan.variant = 0;
        }
    }
    return launch<OutT>(type_idx, plan, p, stream, fixed);
}

template<class T, class U>
constexpr int type_index()
{
    if(std::is_same<T, half>::value && std::is_same<U, half>::value)
        return 0;
    if(std::is_same<T, float>::value && std::is_same<U, half>::value)
        return 1;
    if(std::is_same<T, __hip_bfloat16>::value && std::is_same<U, __hip_bfloat16>::value)
        return 2;
    if(std::is_same<T, float>::value && std::is_same<U, __hip_bfloat16>::value)
        return 3;
    return -1;
}

int run_by_type(int type_idx, const launch_plan* forced, void* C, void* A, void* B, size_t M,
                size_t N, size_t K, size_t batch, int lc, int la, int lb, hipStream_t stream,
                const fixed_scratch* fixed = nullptr)
{
    switch(type_idx)
    {
        case 0: return run<_Float16>(0, forced, C, A, B, M, N, K, batch, lc, la, lb, stream, fixed);
        case 1: return run<float>(1, forced, C, A, B, M, N, K, batch, lc, la, lb, stream, fixed);
        case 2: return run<__bf16>(2, forced, C, A, B, M, N, K, batch, lc, la, lb, stream, fixed);
        case 3: return run<float>(3, forced, C, A, B, M, N, K, batch, lc, la, lb, stream, fixed);
        default: return ROCM_WMMA_GEMM_ERR_ARGUMENT;
    }
}

// The same, for callers that take a status code instead of an exception (the entry points
// that return int): a problem beyond the library's size limits, or a kernel that is not
// there, becomes ROCM_WMMA_GEMM_ERR_LIMIT, and a launch of this call that the runtime rejected
// ROCM_WMMA_GEMM_ERR_RUNTIME (an error that somebody else's earlier call left pending in the
// runtime does not count, and stays pending for its owner).
int run_with_status(int type_idx, const launch_plan* forced, void* C, void* A, void* B, size_t M,
                    size_t N, size_t K, size_t batch, int lc, int la, int lb, hipStream_t stream,
                    const fixed_scratch* fixed)
{
    int rc;
    launch_failure = hipSuccess; // what this call's own launches return is collected here
    try
    {
        rc = run_by_type(type_idx, forced, C, A, B, M, N, K, batch, lc, la, lb, stream, fixed);
    }
    catch(const std::exception&)
    {
        return ROCM_WMMA_GEMM_ERR_LIMIT;
    }
    if(rc == 0 && launch_failure != hipSuccess)
    {
        rc = ROCM_WMMA_GEMM_ERR_RUNTIME;
    }
    return rc;
}

// Scratch memory of the entry point that allocates nothing: one array per GPU, part of
// the library's code object, so it is there from the moment the library is loaded on a
// device until the process ends.  In host code the array's name only stands in for the
// symbol; the memory's address on a device comes from hipGetSymbolAddress, asked once per
// device with that device current, and only that address is ever handed to kernels.
__attribute__((used)) static __device__ __align__(256) unsigned char scratch[ROCM_WMMA_GEMM_NOALLOC_SCRATCH_BYTES];
std::mutex scratch_mutex;
char*      scratch_address[max_devices] = {};

int scratch_of_current_device(fixed_scratch* out)
{
    int dev = -1;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= max_devices)
    {
        return ROCM_WMMA_GEMM_ERR_RUNTIME;
    }
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if(scratch_address[dev] == nullptr)
    {
        void* p = nullptr;
        if(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr)
        {
            (void)hipGetLastError();
            return ROCM_WMMA_GEMM_ERR_RUNTIME;
        }
        scratch_address[dev] = static_cast<char*>(p);
    }
    out->ptr   = scratch_address[dev];
    out->bytes = ROCM_WMMA_GEMM_NOALLOC_SCRATCH_BYTES;
    return 0;
}

} // namespace
} // namespace host

// ---------------------------------------------------------------------------
// C++ API (reference gemm.hpp:50-73, src/gemm.cpp:8-53)
// ---------------------------------------------------------------------------
template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
__host__ void
    gemm(T* C, U* A, U* B, size_t M, size_t N, size_t K, size_t batch_count, hipStream_t& stream)
{
    constexpr int type_idx = host::type_index<T, U>();
    static_assert(type_idx >= 0, "unsupported type pair");
    host::run_by_type(type_idx,
                      nullptr,
                      C,
                      A,
                      B,
                      M,
                      N,
                      K,
                      batch_count,
                      static_cast<int>(layout_C),
                      static_cast<int>(layout_A),
                      static_cast<int>(layout_B),
                      stream);
}

template<m_layout layout_C, m_layout layout_A, m_layout layout_B, class T, class U>
__host__ void gemm(T* C, U* A, U* B, size_t M, size_t N, size_t K, hipStream_t& stream)
{
    gemm<layout_C, layout_A, layout_B, T, U>(C, A, B, M, N, K, size_t{1}, stream);
}

#define ROCM_WMMA_GEMM_INSTANTIATE(LC, LA, LB, T, U)                                          \
    template void gemm<LC, LA, LB, T, U>(T*, U*, U*, size_t, size_t, size_t, hipStream_t&);   \
    template void gemm<LC, LA, LB, T, U>(T*, U*, U*, size_t, size_t, size_t, size_t,          \
                                         hipStream_t&);
ROCM_WMMA_GEMM_FOR_EACH_TYPE_PAIR(ROCM_WMMA_GEMM_INSTANTIATE)
#undef ROCM_WMMA_GEMM_INSTANTIATE

} // namespace rocm_wmma_gemm

// ---------------------------------------------------------------------------
// C ABI (reference src/gemm.cpp:207-250)
// ---------------------------------------------------------------------------
namespace
{
inline hipStream_t stream_of(void* stream)
{
    return stream ? *static_cast<hipStream_t*>(stream) : nullptr;
}
} // namespace

extern "C" {

void rocm_wmma_gemm_f16_f16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                            size_t batch_count, int layout_c, int layout_a, int layout_b,
                            void* stream)
{
    rocm_wmma_gemm::host::run_by_type(
        0, nullptr, C, A, B, M, N, K, batch_count, layout_c, layout_a, layout_b, stream_of(stream));
}

void rocm_wmma_gemm_f32_f16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                            size_t batch_count, int layout_c, int layout_a, int layout_b,
                            void* stream)
{
    rocm_wmma_gemm::host::run_by_type(
        1, nullptr, C, A, B, M, N, K, batch_count, layout_c, layout_a, layout_b, stream_of(stream));
}

void rocm_wmma_gemm_bf16_bf16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                              size_t batch_count, int layout_c, int layout_a, int layout_b,
                              void* stream)
{
    rocm_wmma_gemm::host::run_by_type(
        2, nullptr, C, A, B, M, N, K, batch_count, layout_c, layout_a, layout_b, stream_of(stream));
}

void rocm_wmma_gemm_f32_bf16(void* C, void* A, void* B, size_t M, size_t N, size_t K,
                             size_t batch_count, int layout_c, int layout_a, int layout_b,
                             void* stream)
{
    rocm_wmma_gemm::host::run_by_type(
        3, nullptr, C, A, B, M, N, K, batch_count, layout_c, layout_a, layout_b, stream_of(stream));
}

const char* rocm_wmma_gemm_arch(void)
{
    return "gfx950";
}

int rocm_wmma_gemm_variant_count(void)
{
    return rocm_wmma_gemm::host::variant_total();
}

int rocm_wmma_gemm_variant_info_get(int variant, rocm_wmma_gemm_variant_info* info)
{
    using namespace rocm_wmma_gemm::host;
    if(variant < 0 || variant >= variant_total() || info == nullptr)
    {
        return -1;
    }
    const variant_desc& v = variant_at(variant);
    info->block_m         = v.block_m;
    info->block_n         = v.block_n;
    info->block_k         = v.block_k;
    info->warps_m         = v.waves_m;
    info->warps_n         = v.waves_n;
    info->warp_tile_m     = v.block_m / v.waves_m / 32;
    info->warp_tile_n     = v.block_n / v.waves_n / 32;
    info->pipeline        = v.pipeline;
    info->lds_bytes       = v.lds_bytes;
    info->threads         = v.threads;
    return 0;
}

int rocm_wmma_gemm_select(size_t M, size_t N, size_t K, int type_idx, int layout_c, int layout_a,
                          int layout_b, int* swizzle, int* split_k)
{
    return rocm_wmma_gemm_select_batched(M, N, K, 1, type_idx, layout_c, layout_a, layout_b,
                                         swizzle, split_k);
}

int rocm_wmma_gemm_select_batched(size_t M, size_t N, size_t K, size_t batch_count, int type_idx,
                                  int layout_c, int layout_a, int layout_b, int* swizzle,
                                  int* split_k)
{
    using namespace rocm_wmma_gemm::host;
    if(type_idx < 0 || type_idx >= num_types || ((layout_c | layout_a | layout_b) & ~1)
       || batch_count == 0)
    {
        return -1;
    }
    const launch_plan plan
        = select_plan(M, N, K, type_idx, layout_c, layout_a, layout_b, batch_count);
    if(swizzle)
    {
        *swizzle = plan.swizzle;
    }
    if(split_k)
    {
        *split_k = plan.split_k;
    }
    return plan.variant;
}

int rocm_wmma_gemm_select_ex(size_t M, size_t N, size_t K, size_t batch_count, int type_idx, int layout_c,
                             int layout_a, int layout_b, int* swizzle, int* split_k, int* touch_ahead)
{
    using namespace rocm_wmma_gemm::host;
    if(type_idx < 0 || type_idx >= num_types || ((layout_c | layout_a | layout_b) & ~1)
       || batch_count == 0)
    {
        return -1;
    }
    const launch_plan plan
        = select_plan(M, N, K, type_idx, layout_c, layout_a, layout_b, batch_count);
    if(swizzle)
    {
        *swizzle = plan.swizzle;
    }
    if(split_k)
    {
        *split_k = plan.split_k;
    }
    if(touch_ahead)
    {
        *touch_ahead = plan.touch;
    }
    return plan.variant;
}

int rocm_wmma_gemm_run_variant(int type_idx, int variant, int swizzle, int split_k, void* C,
                               void* A, void* B, size_t M, size_t N, size_t K,
                               size_t batch_count, int layout_c, int layout_a, int layout_b,
                               void* stream)
{
    return rocm_wmma_gemm_run_variant_ex(type_idx, variant, swizzle, split_k, 0, C, A, B, M, N, K,
                                         batch_count, layout_c, layout_a, layout_b, stream);
}

int rocm_wmma_gemm_run_variant_ex(int type_idx, int variant, int swizzle, int split_k, int touch_ahead,
                                  void* C, void* A, void* B, size_t M, size_t N, size_t K,
                                  size_t batch_count, int layout_c, int layout_a, int layout_b,
                                  void* stream)
{
    using namespace rocm_wmma_gemm::host;
    if(type_idx < 0 || type_idx >= num_types || variant < 0 || variant >= variant_total())
    {
        return ROCM_WMMA_GEMM_ERR_ARGUMENT;
    }
    launch_plan plan;
    plan.variant = variant;
    plan.swizzle = swizzle;
    plan.split_k = split_k;
    plan.touch   = touch_ahead < 0 ? 0 : touch_ahead & 0x3ff;
    return run_with_status(type_idx, &plan, C, A, B, M, N, K, batch_count, layout_c, layout_a,
                           layout_b, stream_of(stream), nullptr);
}

int rocm_wmma_gemm_register_variant(int block_m, int block_n, int block_k, int warps_m, int warps_n,
                                    int pipeline, int type_idx, int a_kmajor, int b_kmajor,
                                    const void* const* kernels)
{
    using namespace rocm_wmma_gemm::host;
    if(block_m <= 0 || block_n <= 0 || block_k <= 0 || warps_m <= 0 || warps_n <= 0 || pipeline < 0
       || pipeline > 7 || 64 * warps_m * warps_n > 1024 || type_idx < 0 || type_idx >= num_types
       || kernels == nullptr || ((a_kmajor | b_kmajor) & ~1)
       || ring_bytes(block_m, block_n, block_k, pipeline) > 160 * 1024)
    {
        return ROCM_WMMA_GEMM_ERR_ARGUMENT;
    }
    if(pipeline == 7)
    {
        // the streaming kernel's own tiles: sides of 16, 32, 64 or 128 (at most 192 together),
        // stages of 128, the wave grid spelling the tile in 32-row units (1 for a 16-wide side)
        auto side_ok = [](int side, int waves) {
            return (side == 16 && waves == 1) || ((side == 32 || side == 64 || side == 128) && side == 32 * waves);
        };
        if(block_k != 128 || block_m + block_n < 48 || block_m + block_n > 192 || !side_ok(block_m, warps_m)
           || !side_ok(block_n, warps_n))
        {
            return ROCM_WMMA_GEMM_ERR_ARGUMENT;
        }
    }
    else if(block_m % (32 * warps_m) != 0 || block_n % (32 * warps_n) != 0)
    {
        return ROCM_WMMA_GEMM_ERR_ARGUMENT;
    }
    std::lock_guard<std::mutex> lock(register_mutex);
    const int count = registered_count.load(std::memory_order_relaxed);
    int       slot  = -1;
    // a compiled variant of this description cannot take kernels; a registered one can
    for(int i = 0; i < num_variants; ++i)
    {
        const variant_desc& v = variant_table[i];
        if(v.block_m == block_m && v.block_n == block_n && v.block_k == block_k && v.waves_m == warps_m
           && v.waves_n == warps_n && v.pipeline == pipeline)
        {
            return ROCM_WMMA_GEMM_ERR_VARIANT;
        }
    }
    for(int i = 0; i < count; ++i)
    {
        const variant_desc& v = registered[i].desc;
        if(v.block_m == block_m && v.block_n == block_n && v.block_k == block_k && v.waves_m == warps_m
           && v.waves_n == warps_n && v.pipeline == pipeline)
        {
            slot = i;
        }
    }
    if(slot < 0)
    {
        if(count >= max_registered)
        {
            return ROCM_WMMA_GEMM_ERR_LIMIT;
        }
        slot                  = count;
        registered[slot].desc = {block_m, block_n, block_k, warps_m, warps_n, pipeline,
                                 ring_bytes(block_m, block_n, block_k, pipeline),
                                 workgroup_threads(warps_m, warps_n, pipeline)};
    }
    for(int mode = 0; mode < num_modes; ++mode)
    {
        registered[slot].kernels[type_idx][a_kmajor][b_kmajor][mode].store(
            reinterpret_cast<kernel_fn>(const_cast<void*>(kernels[mode])), std::memory_order_release);
    }
    if(slot == count)
    {
        registered_count.store(count + 1, std::memory_order_release);
    }
    return num_variants + slot;
}

int rocm_wmma_gemm_workspace_release(void)
{
    using namespace rocm_wmma_gemm::host;
    int dev = -1;
    if(hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= max_devices)
    {
        return ROCM_WMMA_GEMM_ERR_RUNTIME;
    }
    std::lock_guard<std::mutex> lock(workspace_mutex);
    if(workspace_ptr[dev] != nullptr && workspace_lent_to_capture[dev])
    {
        return 1; // a captured graph may hold its address
    }
    (void)hipDeviceSynchronize();
    // (nothing of the library is in flight now) the arrival counters of shared tiles go back
    // to zero as well, whatever an aborted kernel may have left in them
    if(unsigned int* counters = arrivals_of_current_device(false))
    {
        (void)hipMemset(counters, 0, stream_arrival_slots * sizeof(unsigned int));
        (void)hipMemset(arrivals_of_current_device(true), 0, stream_arrival_slots * sizeof(unsigned int));
    }
    if(workspace_ptr[dev] == nullptr)
    {
        return 0;
    }
    (void)hipFree(workspace_ptr[dev]);
    workspace_ptr[dev]  = nullptr;
    workspace_size[dev] = 0;
    workspace_used[dev] = false;
    return 0;
}

int rocm_wmma_gemm_noalloc(int type_idx, void* C, void* A, void* B, size_t M, size_t N, size_t K,
                           size_t batch_count, int layout_c, int layout_a, int layout_b,
                           void* stream)
{
    using namespace rocm_wmma_gemm::host;
    if(type_idx < 0 || type_idx >= num_types || ((layout_c | layout_a | layout_b) & ~1))
    {
        return ROCM_WMMA_GEMM_ERR_ARGUMENT;
    }
    fixed_scratch own;
    const int     rc = scratch_of_current_device(&own);
    if(rc != 0)
    {
        return rc;
    }
    return run_with_status(type_idx, nullptr, C, A, B, M, N, K, batch_count, layout_c, layout_a,
                           layout_b, stream_of(stream), &own);
}

} // extern "C"
