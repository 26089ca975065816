// C-ABI entry points of libmxmoe_amd.so.  The kernels of the library are registered by the translation unit that
// mxmoe_amd.kernels.compose_kernel.emit_default_library writes (generated/default_*.hip, one per kernel); generated libraries register
// their own sets and include the same entry points.
#include "include/mxmoe_abi_impl.hpp"
