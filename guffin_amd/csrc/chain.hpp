// Recorded launch chains: the kernels a caller enqueues on a stream between chain_begin and chain_end are
// not run but recorded (kernel, grid, arguments), and every later chain_launch replays them as AQL
// dispatch packets written straight into a hardware queue of the library's own.
//
// Role in the reference: MetalCommandContext encodes a whole pass into one command buffer and commits it
// once (src/tensor/backends/metal/metal_command_context.hpp:346-353); a chain is that command buffer.
// What it adds over a HIP graph of the same launches is control over the packet header: a kernel that
// keeps its own order with its predecessor (a counter the predecessor's workgroups raise when their
// stores have landed, polled with a bound by the successor's workgroups) is dispatched without the
// packet barrier, so its workgroups become resident while the predecessor drains and their first weight
// tiles travel during the hand-over.  Such kernels take a ChainLink; everything else is dispatched with
// the barrier and agent-scope fences, exactly like a stream.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstring>
#include <utility>

namespace guffin {

// What a chained kernel needs to order itself: it waits until counters[wait_index * 32] has reached
// wait_count (nothing to wait for when wait_count is 0), and every workgroup adds one to
// counters[signal_index * 32] after its stores have completed (no signal when counters is null).
struct ChainLink {
    uint32_t* counters;
    uint32_t wait_index, wait_count, signal_index, spin_limit;
    uint32_t* status;
};

namespace chain {

struct Recorder;

// the recorder bound to `stream`, or null when launches on it run as usual
Recorder* recorder_for(hipStream_t stream);
// appends one launch; `chained`: the kernel follows the ChainLink protocol with `link` (already part of `args`)
void record(Recorder* r, const void* host_function, dim3 grid, dim3 block, uint32_t lds_bytes, const void* args,
            uint32_t arg_bytes, bool chained);
// the link of the next chained launch: waits for the previous launch if that was chained too, signals its own
// counter with `arrivals` workgroups; a null recorder gives the inert link
ChainLink next_link(Recorder* r, uint32_t arrivals, uint32_t* status);

template <typename T>
inline void pack(uint8_t* buf, size_t& off, const T& v) {
    off = (off + alignof(T) - 1) & ~(alignof(T) - 1);
    std::memcpy(buf + off, &v, sizeof(T));
    off += sizeof(T);
}

}  // namespace chain

// Launches `kernel` on `stream`, or records the launch when the stream is being recorded.  Arguments are laid out
// as the kernel's parameter list lays them out (natural alignment, in order): the layout of a kernarg segment.
template <typename... P, typename... A>
inline void launch_on(bool chained, void (*kernel)(P...), dim3 grid, dim3 block, uint32_t lds_bytes, hipStream_t stream, A&&... args) {
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    if (chain::Recorder* r = chain::recorder_for(stream)) {
        alignas(16) uint8_t buf[4096];
        size_t off = 0;
        (chain::pack<P>(buf, off, static_cast<P>(args)), ...);
        static_assert((sizeof(P) + ... + 0) <= 3584, "kernel arguments exceed the staging buffer");
        chain::record(r, reinterpret_cast<const void*>(kernel), grid, block, lds_bytes, buf, static_cast<uint32_t>(off), chained);
        return;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, std::forward<A>(args)...);
}

template <typename... P, typename... A>
inline void launch(void (*kernel)(P...), dim3 grid, dim3 block, uint32_t lds_bytes, hipStream_t stream, A&&... args) {
    launch_on(false, kernel, grid, block, lds_bytes, stream, std::forward<A>(args)...);
}

}  // namespace guffin
