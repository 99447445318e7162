// What a call that needs library-owned scratch memory may do with the per-device buffer.
// Pure (no HIP calls), so the rules can be tested on the host; gemm.hip carries them out.
//
// The rules exist because a stream under graph capture bakes the buffer's address into
// the graph, and because nothing that allocates, frees or synchronises may run while a
// stream is capturing:
//   - a call on a capturing stream takes the buffer only as it is; when the buffer is
//     missing or too small the call gets nothing and runs without scratch memory;
//   - a buffer that was ever handed to a capturing stream is never freed: when a later
//     call outgrows it, the old buffer is retired (kept allocated for the replays of
//     graphs that hold its address) and a new one takes its place.
// The reference needs no such rules: it has no workspace at all (reference
// rocm_wmma_gemm/src/gemm.cpp:14-53 launches one kernel and owns nothing).
#ifndef ROCM_WMMA_GEMM_WORKSPACE_POLICY_HPP
#define ROCM_WMMA_GEMM_WORKSPACE_POLICY_HPP

#include <cstddef>

namespace rocm_wmma_gemm
{
namespace host
{

enum class workspace_action
{
    use_existing, // the buffer is large enough
    allocate, // there is no buffer yet: allocate one
    grow_free_old, // synchronise the device, free the buffer, allocate a larger one
    grow_retire_old, // keep the buffer allocated for captured graphs, allocate a larger one
    refuse // the call gets no scratch memory
};

inline workspace_action workspace_decide(size_t have_bytes, size_t need_bytes, size_t limit_bytes,
                                         bool stream_is_capturing, bool lent_to_a_capture)
{
    if(need_bytes > limit_bytes)
    {
        return workspace_action::refuse;
    }
    if(have_bytes >= need_bytes && have_bytes > 0)
    {
        return workspace_action::use_existing;
    }
    if(stream_is_capturing)
    {
        return workspace_action::refuse;
    }
    if(have_bytes == 0)
    {
        return workspace_action::allocate;
    }
    return lent_to_a_capture ? workspace_action::grow_retire_old : workspace_action::grow_free_old;
}

// Size of a new buffer for a call that needs need_bytes: a quarter more than asked, so
// that a slowly growing sequence of calls does not reallocate every time, and never less
// than first_bytes.
inline size_t workspace_grown_size(size_t need_bytes, size_t first_bytes)
{
    const size_t want = need_bytes + need_bytes / 4;
    return want > first_bytes ? want : first_bytes;
}

} // namespace host
} // namespace rocm_wmma_gemm

#endif
