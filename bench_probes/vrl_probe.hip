// libvrl_probe.so: host launchers of the bench-side probes declared in vrl_probe.h.
#include "vrl_probe.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "vrl.h"

#include "probe_kernels.h"
#include "row_shapes.h"

namespace {

constexpr int64_t kMaxGrid = 0x7fffffffLL;

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

int launch_status() { return hipGetLastError() == hipSuccess ? VRL_OK : VRL_ERR_HIP; }

}  // namespace

extern "C" {

int vrl_stream_probe(const void* src, void* dst, int64_t n_rows, int64_t row_bytes, int mode, uint32_t* sink,
                     void* stream) {
  if (mode < 0 || mode > 4) return VRL_ERR_ARG;
  if (n_rows < 0 || row_bytes < 0 || row_bytes % 16 != 0 || n_rows > kMaxGrid) return VRL_ERR_SHAPE;
  if (n_rows == 0 || row_bytes == 0) return VRL_OK;
  const bool reads_only = mode == 0 || mode == 3 || mode == 4;
  if (src == nullptr || (!reads_only && dst == nullptr) || (reads_only && sink == nullptr)) return VRL_ERR_NULL;
  if (!aligned(src, 16) || !aligned(dst, 16) || !aligned(sink, 4)) return VRL_ERR_ALIGN;
  const dim3 grid(static_cast<unsigned>(n_rows));
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t vecs = row_bytes / 16;
  // the forward / backward row kernels' workgroup shapes for 16-bit logits
  if (mode == 0)
    vrl::stream_probe_kernel<RowShape<VRL_BF16>::kWaves, RowShape<VRL_BF16>::kUnroll, false>
        <<<grid, dim3(RowShape<VRL_BF16>::kWaves * 64), 0, s>>>(static_cast<const vrl::u32x4*>(src), nullptr, vecs,
                                                                0x9e3779b9u, sink);
  else if (mode == 3)   // the forward kernel's workgroup shape for 32-bit logits
    vrl::stream_probe_kernel<RowShape<VRL_F32>::kWaves, RowShape<VRL_F32>::kUnroll, false>
        <<<grid, dim3(RowShape<VRL_F32>::kWaves * 64), 0, s>>>(static_cast<const vrl::u32x4*>(src), nullptr, vecs,
                                                               0x9e3779b9u, sink);
  else if (mode == 1)
    vrl::stream_probe_kernel<kBackwardWaves, kBackwardUnroll, true><<<grid, dim3(kBackwardWaves * 64), 0, s>>>(
        static_cast<const vrl::u32x4*>(src), static_cast<vrl::u32x4*>(dst), vecs, 0u, nullptr);
  else if (mode == 4)
    vrl::stream_probe_flat_read_kernel<<<dim3(1024), dim3(256), 0, s>>>(static_cast<const vrl::u32x4*>(src),
                                                                        n_rows * vecs, 0x9e3779b9u, sink);
  else
    vrl::stream_probe_flat_copy_kernel<<<dim3(512), dim3(256), 0, s>>>(
        static_cast<const vrl::u32x4*>(src), static_cast<vrl::u32x4*>(dst), n_rows * vecs);
  return launch_status();
}

int vrl_mfma_probe(int64_t n_workgroups, int64_t iters, int instruction, int random_operands, float* sink,
                   int64_t* clocks, int64_t* wall_clock_khz, void* stream) {
  if (n_workgroups < 0 || iters < 0 || n_workgroups > kMaxGrid) return VRL_ERR_SHAPE;
  if (iters > VRL_PROBE_MAX_ITERS) return VRL_ERR_ARG;   // an unbounded loop on every CU is no measurement
  if (instruction != 16 && instruction != 32) return VRL_ERR_ARG;
  if (wall_clock_khz != nullptr) {
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) {
      (void)hipGetLastError();
      return VRL_ERR_HIP;
    }
    *wall_clock_khz = khz;
  }
  if (n_workgroups == 0) return VRL_OK;
  if (sink == nullptr) return VRL_ERR_NULL;
  if (!aligned(sink, 4) || !aligned(clocks, 8)) return VRL_ERR_ALIGN;
  const dim3 grid(static_cast<unsigned>(n_workgroups));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (instruction == 16)
    vrl::mfma_probe_kernel<16><<<grid, dim3(512), 0, s>>>(iters, random_operands != 0 ? 1 : 0, sink, clocks);
  else
    vrl::mfma_probe_kernel<32><<<grid, dim3(512), 0, s>>>(iters, random_operands != 0 ? 1 : 0, sink, clocks);
  return launch_status();
}

}  // extern "C"
