// int8 instantiations of the convolution kernels.
#include "scn_conv_kernels.hpp"

namespace scn {

bool conv_dispatch_int8(const ConvWeights& w, uint32_t n_hint, ConvArgs& a, hipStream_t stream) {
  bool ok = false;
  const int mt32 = w.mtiles32;
  if (a.tmask && conv_tile_covers(w) && dispatch_tile<0>(w.chunks, mt32, n_hint, a, stream)) return true;
  if (mt32 >= 1 && mt32 <= 4 && conv_impl() == 0) {
    a.wfrag = w.wfrag32.as<uint4>();
    ok = dispatch_chunks32<0>(w.chunks, mt32, n_hint, a, stream);
  }
  if (!ok) {
    a.wfrag = w.wfrag.as<uint4>();
    ok = dispatch_chunks<0>(w.chunks, w.mtiles, a, stream);
  }
  return ok;
}

}  // namespace scn
