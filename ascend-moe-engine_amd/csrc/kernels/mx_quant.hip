// Standalone block-32 MX quantisation of bf16 rows: the operator behind the reference's stages
// `attn_quant` and `shared_act_quant` (aclnnDynamicMxQuant, src/pipeline/pipeline.cpp:251-258).
// HBM-bound: 2 bytes read, 1 + 1/32 written per element.
#include "kernels.h"
#include "mx_quant_device.h"

namespace mlakv {
namespace {

typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// A thread takes 8 consecutive values (16 bytes); the four threads of a block of 32 are
// neighbouring lanes of one wavefront (cols is a multiple of 32, so blocks never straddle rows).
__global__ __launch_bounds__(256) void MxQuantKernel(MxQuantArgs q) {
  const int64_t item = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int items_per_row = q.cols >> 3;
  const int64_t row = item / items_per_row;
  const bool live = row < q.rows;  // dead lanes still take part in the shuffles
  const int col8 = static_cast<int>(item - row * items_per_row);
  u32x4 v = {0u, 0u, 0u, 0u};
  if (live) v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(q.x + row * q.x_row_stride + col8 * 16));
  unsigned magnitude = 0u;
#pragma unroll
  for (int i = 0; i < 4; ++i) magnitude = MxMagnitudeMax(v[i], magnitude);
  magnitude = max(magnitude, static_cast<unsigned>(__shfl_xor(static_cast<int>(magnitude), 1)));
  magnitude = max(magnitude, static_cast<unsigned>(__shfl_xor(static_cast<int>(magnitude), 2)));
  if (!live) return;
  const MxScale s = MxScaleFromMaxBits(magnitude);
  u32x2 codes;
  codes.x = MxEncodeWord(v[0], s) | (MxEncodeWord(v[1], s) << 16);
  codes.y = MxEncodeWord(v[2], s) | (MxEncodeWord(v[3], s) << 16);
  __builtin_nontemporal_store(codes, reinterpret_cast<u32x2*>(q.codes + row * q.codes_row_stride + col8 * 8));
  if ((col8 & 3) == 0) reinterpret_cast<unsigned char*>(q.scales + row * q.scales_row_stride)[col8 >> 2] = static_cast<unsigned char>(s.code);
}

}  // namespace

hipError_t PrepareMxQuantKernels() {
  hipFuncAttributes attributes;  // (no attribute to set: the call only loads the kernel onto the current device)
  return hipFuncGetAttributes(&attributes, reinterpret_cast<const void*>(&MxQuantKernel));
}

hipError_t LaunchMxQuant(const MxQuantArgs& args, hipStream_t stream) {
  if (args.rows <= 0 || args.cols <= 0) return hipSuccess;
  const int64_t items = args.rows * (args.cols >> 3);
  const int64_t groups = (items + 255) / 256;
  if (groups > 0x7fffffff) return hipErrorInvalidValue;
  hipLaunchKernelGGL(MxQuantKernel, dim3(static_cast<unsigned>(groups)), dim3(256), 0, stream, args);
  return hipGetLastError();
}

}  // namespace mlakv
