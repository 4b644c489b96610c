// Entry points of the window-resident attention kernels that run on 16-bit matrix-core operands
// (window_attention_x16.hip).  Arguments are checked by the callers in window_attention.hip.
#pragma once

#include "wattn_common.hpp"

namespace sswin {
namespace x16 {

void forward(int dtype, const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
             const TokenTensor32& o, float* lse, hipStream_t s);
void backward(int dtype, const WAttnCommon& a, const TokenTensor32& q, const TokenTensor32& k, const TokenTensor32& v,
              const TokenTensor32& o, const TokenTensor32& d_o, const float* lse, const TokenTensor32& dq,
              const TokenTensor32& dk, const TokenTensor32& dv, float* ds_out, int sides, hipStream_t s);

}  // namespace x16
}  // namespace sswin
