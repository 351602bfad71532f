// Kernel launch that reports the status of that launch and of nothing else.
//
// `kernel<<<...>>>(...)` followed by hipGetLastError() reads (and clears) the
// calling thread's last-error slot, which an unrelated earlier call may have
// filled; hipLaunchKernel returns the status of the launch it makes and leaves
// that slot alone on success.
#ifndef NVJ_LAUNCH_H_
#define NVJ_LAUNCH_H_

#include <hip/hip_runtime.h>

#include <type_traits>

namespace nvj {

// Arguments are converted to the kernel's parameter types (the parameter pack
// is deduced from the kernel alone) and handed over by address.
template <typename... Params>
inline hipError_t launch(void (*kernel)(Params...), dim3 grid, dim3 block, hipStream_t stream,
                         typename std::common_type<Params>::type... args) {
  void* ptrs[] = {static_cast<void*>(&args)..., nullptr};
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, 0, stream);
}

}  // namespace nvj

#endif  // NVJ_LAUNCH_H_
