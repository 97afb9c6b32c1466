// Instances of the direct-to-LDS contraction kernel (gemm_dtl.hpp), in a translation unit of their own
// so that they compile beside the register-staged kernels of gemm.hip.
#include <hip/hip_runtime.h>

#include "gemm.hpp"
#include "gemm_common.hpp"
#include "gemm_dtl.hpp"

namespace ocannl {
namespace {

template <int BM, int BN, int BK, int NS>
hipError_t launch_dtl_layout(bool akc, bool bkc, const GemmArgs& a, hipStream_t s, hipEvent_t ev) {
  constexpr size_t smem = dtl_smem<BM, BN, BK, NS>();
  if (akc && bkc) return launch(gemm_bf16_dtl_kernel<BM, BN, BK, NS, true, true>, smem, BM, BN, a, s, ev);
  if (akc && !bkc) return launch(gemm_bf16_dtl_kernel<BM, BN, BK, NS, true, false>, smem, BM, BN, a, s, ev);
  if (!akc && bkc) return launch(gemm_bf16_dtl_kernel<BM, BN, BK, NS, false, true>, smem, BM, BN, a, s, ev);
  return launch(gemm_bf16_dtl_kernel<BM, BN, BK, NS, false, false>, smem, BM, BN, a, s, ev);
}


}  // namespace

hipError_t launch_gemm_dtl(int bm, int bn, int bk, int ns, bool akc, bool bkc, const GemmArgs& a, hipStream_t s, hipEvent_t ev) {
  if (bm == 256 && bn == 256 && bk == 32 && ns == 4) return launch_dtl_layout<256, 256, 32, 4>(akc, bkc, a, s, ev);
  if (bm == 128 && bn == 64 && bk == 32 && ns == 4) return launch_dtl_layout<128, 64, 32, 4>(akc, bkc, a, s, ev);
  if (bm == 128 && bn == 128 && bk == 64 && ns == 5) return launch_dtl_layout<128, 128, 64, 5>(akc, bkc, a, s, ev);
  if (bm == 128 && bn == 128 && bk == 32 && ns == 4) return launch_dtl_layout<128, 128, 32, 4>(akc, bkc, a, s, ev);
  return hipErrorInvalidValue;
}

}  // namespace ocannl
