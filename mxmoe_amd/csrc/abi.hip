// C-ABI entry points of libmxmoe_amd.so and the default set of fused kernels.
#include "include/mxmoe_abi_impl.hpp"

namespace {

// Default fused kernels.  Generated libraries (mxmoe_amd.kernels.compose_kernel) register their own sets.
struct DefaultKernels {
  DefaultKernels() {
    register_fused<WxAxTile<Op::I4, 128, 256>, WxAxTile<Op::I4, 64, 256>, WxAxTile<Op::I4, 32, 256>,
                   WxAxTile<Op::I8, 128, 256>, WxAxTile<Op::I8, 64, 256>, WxAxTile<Op::I8, 32, 256>>("groupgemm_hz_fused_wxax");
    register_fused<MfmaTile<Op::F16, 128, 256, 2, 2>, MfmaTile<Op::F16, 64, 256, 1, 4>, MfmaTile<Op::F16, 32, 256, 1, 4>>("groupgemm_hz_fused_fp16");
    register_fused<SkinnyWoTile<4, 128>, SkinnyWoTile<3, 128>, SkinnyWoTile<2, 128>, WoMfmaTile<4>, WoMfmaTile<3>, WoMfmaTile<2>>("groupgemm_hz_fused_wo");
    register_fused<WxAxGTile<64>, WxAxGTile<32>>("groupgemm_hz_fused_wxax_g128");
    // every format in one launch (layers that mix weight-only, w-a and fp16 blocks)
    register_fused<WxAxTile<Op::I4, 128, 256>, WxAxTile<Op::I4, 32, 256>, WxAxTile<Op::I8, 128, 256>, WxAxTile<Op::I8, 32, 256>,
                   MfmaTile<Op::F16, 128, 256, 2, 2>, MfmaTile<Op::F16, 32, 256, 1, 4>, SkinnyWoTile<4, 128>, SkinnyWoTile<3, 128>, SkinnyWoTile<2, 128>, WoMfmaTile<4>, WoMfmaTile<3>, WoMfmaTile<2>, WxAxGTile<64>>("groupgemm_hz_fused_all");
  }
};
DefaultKernels g_default_kernels;

}  // namespace

