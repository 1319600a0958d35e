// The launch interface of libtm_hip: everything the host logic (tm_hip.cpp) asks
// of the device beyond the HIP runtime API itself. tm_launch.cpp implements it
// with the gfx950 kernels; the CPU build of the host logic links a recording
// stand-in instead, which is how the planner, the leases and the commit
// bookkeeping run under sanitizers without a GPU.
#pragma once

#include <hip/hip_runtime.h>

#include "tm_plan.hpp"

namespace tmdev {

// hipSuccess when the device code for the current device is present (asked once
// at context creation, so that a missing code object fails there and not at the
// first product).
hipError_t kernels_present();

// This device's address of the static workspace of tm_hip_q8_0_gemm_mma_noalloc
// (tmh::kScratchBytes, layout in tm_plan.hpp), asked once per device with that
// device current.
hipError_t scratch_on_current_device(int device, uint8_t **out);

// A planned launch of a product list (tmh::Launch::single == nullptr) on `stream`;
// `stop`, when not null, completes with the launch's last kernel. `ws`: the
// workspace the kernels may use beyond the products' own buffers.
hipError_t launch_list(hipStream_t stream, hipEvent_t stop, const tmh::Launch &launch,
                       const tmh::Workspace &ws);

// A single operation. `split_to`: where an RMSNorm or gated activation writes the
// split form of its result as well, or null. `update`: a residual update
// h += alpha * t that an RMSNorm of h takes in front of itself, or null.
hipError_t launch_single(hipStream_t stream, hipEvent_t stop, const tmh::Op &op, uint16_t *split_to,
                         uint32_t split_cols, const tmh::Op *update);

// dst[0 .. n) = 0 with a fill kernel (not a memset node: the caller may be recording).
hipError_t zero_words(hipStream_t stream, uint32_t *dst, uint32_t n);

} // namespace tmdev
