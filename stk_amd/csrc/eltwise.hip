// stk_activation_product: an activation (or its derivative) of stored 16-bit sums times a second array, element by
// element - the step of a backward pass that stk_sdd_fused_sums makes possible: with the sums of the forward product
// kept, the gradient with respect to them is act'(sums) * incoming gradient, one pass over the values instead of a
// product that computes the sums again.  Same arithmetic as the store of stk_sdd_fused: the function in fp32, rounded,
// then the product of the two 16-bit values rounded once more; a derivative times its factor is rounded once.
#include "common.h"
#include "gemm_core.h"

namespace stk {

__device__ __forceinline__ float activate_one(float x, int kind) {
  switch (kind) {
    case kRelu: return activate<kRelu>(x);
    case kGeluTanh: return activate<kGeluTanh>(x);
    case kGeluErf: return activate<kGeluErf>(x);
    case kSilu: return activate<kSilu>(x);
    case kReluGrad: return activate<kReluGrad>(x);
    case kGeluTanhGrad: return activate<kGeluTanhGrad>(x);
    case kGeluErfGrad: return activate<kGeluErfGrad>(x);
    case kSiluGrad: return activate<kSiluGrad>(x);
    default: return x;
  }
}

// One 16-byte piece (eight values) per thread and trip.
template <bool BF16>
__global__ __launch_bounds__(256) void activation_product_kernel(const u32x4* __restrict__ sums, const u32x4* __restrict__ factor,
                                                                 u32x4* __restrict__ out, int64_t pieces, int activation) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < pieces; i += stride) {
    const u32x4 s = __builtin_nontemporal_load(sums + i);
    u32x4 f = {0u, 0u, 0u, 0u};
    if (factor) f = __builtin_nontemporal_load(factor + i);
    uint32_t v[4] = {s.x, s.y, s.z, s.w};
    const uint32_t fs[4] = {f.x, f.y, f.z, f.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const f32x2_t x = unpack2<BF16>(v[j]);
      const float lo = activate_one(x.x, activation), hi = activate_one(x.y, activation);
      if (factor && activation >= kReluGrad) {
        const f32x2_t y = unpack2<BF16>(fs[j]);
        v[j] = pack2<BF16>(lo * y.x, hi * y.y);
      } else {
        v[j] = pack2<BF16>(lo, hi);
        if (factor) v[j] = mul_packed<BF16>(v[j], fs[j]);
      }
    }
    __builtin_nontemporal_store(u32x4{v[0], v[1], v[2], v[3]}, out + i);
  }
}

}  // namespace stk

extern "C" int stk_activation_product(const void* sums, const void* factor, void* out, int64_t count, int activation, int dtype,
                                      stk_stream_t stream) {
  using namespace stk;
  const char* who = "stk_activation_product";
  if (dtype != STK_F16 && dtype != STK_BF16) return fail(STK_ERR_UNSUPPORTED, "%s: dtype %d", who, dtype);
  if (activation < 0 || activation >= kActivations) return fail(STK_ERR_UNSUPPORTED, "%s: activation %d", who, activation);
  if (count < 0 || count % 8) return fail(STK_ERR_DIMS, "%s: %lld values (a multiple of 8: whole blocks)", who, (long long)count);
  if (count == 0) return STK_OK;
  if (!sums || !out || !aligned16(sums) || !aligned16(out) || !aligned16(factor))
    return fail(STK_ERR_UNSUPPORTED, "%s: arrays need 16-byte aligned bases", who);
  const int64_t pieces = count / 8;
  const int cus = compute_units();
  const int64_t want = (pieces + 255) / 256, most = (int64_t)(cus > 0 ? cus : 256) * 16;
  const int grid = (int)(want < most ? want : most);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == STK_BF16)
    hipLaunchKernelGGL((activation_product_kernel<true>), dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(sums),
                       static_cast<const u32x4*>(factor), static_cast<u32x4*>(out), pieces, activation);
  else
    hipLaunchKernelGGL((activation_product_kernel<false>), dim3(grid), dim3(256), 0, s, static_cast<const u32x4*>(sums),
                       static_cast<const u32x4*>(factor), static_cast<u32x4*>(out), pieces, activation);
  return check_launch(who);
}
