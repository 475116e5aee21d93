// Recorded launch chains: the kernels a caller enqueues on a stream between chain_begin and chain_end are
// not run but recorded (kernel, grid, arguments), and every later chain_launch replays them as AQL
// dispatch packets written straight into a hardware queue of the library's own.
//
// Role in the reference: MetalCommandContext encodes a whole pass into one command buffer and commits it
// once (src/tensor/backends/metal/metal_command_context.hpp:346-353); a chain is that command buffer.
// Every packet carries the barrier bit and agent-scope fences, the last one a system-scope release and
// the completion signal: the order and visibility a stream gives, at the same cost per kernel as a HIP
// graph replay (1.5 us for an empty kernel on this part; packets without the barrier, with kernels that
// order themselves through counters and device-coherent accesses, were built and measured slower:
// every hand-over through memory costs more than the packet processor's own barrier).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstring>
#include <utility>

namespace guffin {

namespace chain {

struct Recorder;

// the recorder bound to `stream`, or null when launches on it run as usual
Recorder* recorder_for(hipStream_t stream);
// appends one launch
void record(Recorder* r, const void* host_function, dim3 grid, dim3 block, uint32_t lds_bytes, const void* args,
            uint32_t arg_bytes);

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
inline void launch(void (*kernel)(P...), dim3 grid, dim3 block, uint32_t lds_bytes, hipStream_t stream, A&&... args) {
    static_assert(sizeof...(P) == sizeof...(A), "one argument per kernel parameter");
    if (chain::Recorder* r = chain::recorder_for(stream)) {
        alignas(16) uint8_t buf[4096];
        size_t off = 0;
        (chain::pack<P>(buf, off, static_cast<P>(args)), ...);
        static_assert((sizeof(P) + ... + 0) <= 3584, "kernel arguments exceed the staging buffer");
        chain::record(r, reinterpret_cast<const void*>(kernel), grid, block, lds_bytes, buf, static_cast<uint32_t>(off));
        return;
    }
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, stream, std::forward<A>(args)...);
}

}  // namespace guffin
