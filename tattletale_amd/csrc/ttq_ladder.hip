// Roofline ladder for the Q4_K decode GEMV: what each stage of the kernel costs on its own.
//
// Not part of libttq_hip.so.  bench.py --only ladder loads libttq_ladder.so, times the rungs with
// the method of the headline row (HIP graph replay over rotated weight copies) and the last rung
// through the product library; a rocprofv3 kernel trace of that command names every rung.
//
//   rung 0  empty kernel: the launch shape of the GEMV (one workgroup of 512 threads per compute
//           unit, its static LDS) and nothing else
//   rung 1  requests only: every wavefront asks for its blocks exactly as the GEMV does (one line of
//           eight rows per global_load_lds_dwordx4, non-temporal), all at once, and waits
//   rung 2  rung 1 and the store of the workgroup's rows of y
//   rung 3  the GEMV without its arithmetic: request schedule, waits, operand reads from LDS and the
//           activation prologue stay
//   (rung 4, the GEMV itself, is ttq_gemv_q4_k of the product library)
//
// The Q6_K streamed GEMV (ttq_gemv_q6k_stream.h) has its stages built in: ttq_ladder_q6k_launch runs it without
// the arithmetic on the operands (stage 1) or without the operand reads as well (stage 2: requests, waits and
// barriers); the GEMV itself is ttq_gemv_q6_k of the product library.
#include "ttq_gemv_q4k_stream.h"
#include "ttq_gemv_q6k_stream.h"

namespace ttq {

int device_num_cus() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess &&
           prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
  }
  return cus;
}

// rungs 0-2: STORE = the y store, REQ = the requests
template <bool REQ, bool STORE>
__global__ void __launch_bounds__(kStThreads)
ladder_kernel(const uint8_t* __restrict__ w, float* __restrict__ y, int n_out, int nsb, int rows_per_wg) {
  __shared__ __attribute__((aligned(1024))) uint8_t wbuf[kStWaves * kStBlockBytes];
  __shared__ uint8_t rest[162832 - kStWaves * kStBlockBytes];   // the GEMV's other tables
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int nks_log2 = nsb >> 4;
  const uint32_t rb = (uint32_t)nsb * 144u;
  const int wg_row0 = blockIdx.x * rows_per_wg;
  const int wg_row_end = min(wg_row0 + rows_per_wg, n_out);
  const int last = wg_row_end - 1;
  const int nblocks = ((wg_row_end - wg_row0 + 15) >> 4) << nks_log2;
  uint8_t* mybuf = wbuf + wave * kStBlockBytes;
  if (REQ) {
    for (int blk = wave; blk < nblocks; blk += kStWaves) {
      const int rg = blk >> nks_log2, ks = blk & ((1 << nks_log2) - 1);
      const int r8 = lane >> 3;
      uint32_t lane_off[2];
#pragma unroll
      for (int o = 0; o < 2; o++) {
        const int row16 = 8 * o + r8;
        const int row = min(wg_row0 + rg * 16 + row16, last);
        lane_off[o] = (uint32_t)row * rb + (uint32_t)(ks * kStSegBytes) + (uint32_t)(((lane & 7) ^ ((row16 >> 1) & 7)) * 16);
      }
#pragma unroll
      for (int i = 0; i < kStBlockRequests; i++) {
        const int line = i >> 1, o = i & 1;
        __builtin_amdgcn_global_load_lds((st_gptr_t)(w + (size_t)(lane_off[o] + (uint32_t)(line * 128))),
                                         (st_lptr_t)(mybuf + o * kStHalfBytes + line * 1024), 16, 0, 2);
      }
      st_wait_vmcnt<0>();
    }
  }
  __syncthreads();
  float v = (float)rest[tid] + (float)wbuf[tid * 16];
  if (STORE) {
    for (int t = tid; t < wg_row_end - wg_row0; t += kStThreads) y[wg_row0 + t] = v;
  } else if (v == 12345.f) {
    y[0] = v;
  }
}

}  // namespace ttq

extern "C" __attribute__((visibility("default")))
int ttq_ladder_launch(int rung, const void* w, const void* x_bf16, float* y, int64_t n_out, int64_t n_in, void* stream) {
  using namespace ttq;
  if (!w || !x_bf16 || !y || (n_in != 2048 && n_in != 4096) || n_out < 16 || rung < 0 || rung > 3) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (rung == 3)
    return st_launch_xy<bf16_tag, float, 1>(w, x_bf16, y, nullptr, 0, 1, n_out, n_in, s) == hipSuccess ? 0 : -7;
  int num_wg = 0;
  const int rows_per_wg = st_rows_per_wg(n_out, &num_wg);
  const dim3 grid((unsigned)num_wg), block(kStThreads);
  const uint8_t* wb = static_cast<const uint8_t*>(w);
  if (rung == 0) hipLaunchKernelGGL((ladder_kernel<false, false>), grid, block, 0, s, wb, y, (int)n_out, (int)(n_in / 256), rows_per_wg);
  if (rung == 1) hipLaunchKernelGGL((ladder_kernel<true, false>), grid, block, 0, s, wb, y, (int)n_out, (int)(n_in / 256), rows_per_wg);
  if (rung == 2) hipLaunchKernelGGL((ladder_kernel<true, true>), grid, block, 0, s, wb, y, (int)n_out, (int)(n_in / 256), rows_per_wg);
  return hipGetLastError() == hipSuccess ? 0 : -7;
}

extern "C" __attribute__((visibility("default")))
int ttq_ladder_q6k_launch(int stage, const void* w, const void* x_bf16, float* y, int64_t n_out, int64_t n_in, void* stream) {
  using namespace ttq;
  if (!w || !x_bf16 || !y || stage < 1 || stage > 2 || !q6_plan(n_out, n_in).ok) return -1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const hipError_t e = stage == 1 ? q6_launch_xy<bf16_tag, float, 1>(w, x_bf16, y, nullptr, 0, 1, n_out, n_in, s)
                                  : q6_launch_xy<bf16_tag, float, 2>(w, x_bf16, y, nullptr, 0, 1, n_out, n_in, s);
  return e == hipSuccess ? 0 : -7;
}
