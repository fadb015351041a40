// One width instance of the whole-plane kernels for small feature maps: compiled once per instance with
//   -DDWCONV_SMALL_W=<width or capacity> -DDWCONV_SMALL_RAG=<0 exact | 1 ragged>
// and, to keep each compile short, once per half: -DDWCONV_SMALL_PART=0 (forward / grad-input kernels,
// dwconv_small_fir.hpp) or 1 (grad-weight and fused backward kernels, dwconv_small_bwd.hpp).
#if !defined(DWCONV_SMALL_W) || !defined(DWCONV_SMALL_RAG) || !defined(DWCONV_SMALL_PART)
#error "compile with -DDWCONV_SMALL_W=.. -DDWCONV_SMALL_RAG=.. -DDWCONV_SMALL_PART=.."
#endif

#if DWCONV_SMALL_PART == 0
#include "dwconv_small_fir.hpp"

namespace dwconv {
#define DWCONV_INSTANTIATE(IO) \
    template int small_fir_width<DWCONV_SMALL_W, DWCONV_SMALL_RAG != 0, IO>(SmallPlan &, int, int, int, bool, bool, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE
}  // namespace dwconv

#else
#include "dwconv_small_bwd.hpp"

namespace dwconv {
#define DWCONV_INSTANTIATE(IO) \
    template long small_bwd_width<DWCONV_SMALL_W, DWCONV_SMALL_RAG != 0, IO>(int, const SmallBwdArgs &, const WgradGeometry &, hipStream_t);
DWCONV_INSTANTIATE(float)
DWCONV_INSTANTIATE(half_t)
DWCONV_INSTANTIATE(bf16_t)
#undef DWCONV_INSTANTIATE
}  // namespace dwconv
#endif
