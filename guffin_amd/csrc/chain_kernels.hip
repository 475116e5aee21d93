// The one kernel the chain engine itself needs: every replay starts by clearing the chain's counters.
#include "common.hpp"

namespace guffin {
namespace {
__global__ void __launch_bounds__(256) chain_clear_kernel(uint32_t* words, uint32_t count) {
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < count) words[i] = 0u;
}
}  // namespace

void chain_clear_counters(hipStream_t stream, uint32_t* counters, uint32_t words) {
    launch(chain_clear_kernel, dim3((words + 255) / 256), dim3(256), 0, stream, counters, words);
}
}  // namespace guffin
