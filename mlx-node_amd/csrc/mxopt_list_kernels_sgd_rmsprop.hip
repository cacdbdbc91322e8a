// mxopt kernels for gfx950, part 4: deferred accumulation for SGD with momentum and RMSprop.
#include "mxopt_list_kernels.h"

namespace mxopt {

bool launch_sgd_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_sgd_hp& hp, const DevPrep& prep) {
  if (od != pd) return false;
  switch (pd) {
    case MXOPT_F32: return update_list_for_pd<MXOPT_F32>(gd, xd, L, SgdMath{hp}, prep);
    case MXOPT_BF16: return update_list_for_pd<MXOPT_BF16>(gd, xd, L, SgdMath{hp}, prep);
    case MXOPT_F16: return update_list_for_pd<MXOPT_F16>(gd, xd, L, SgdMath{hp}, prep);
  }
  return false;
}

bool launch_rmsprop_list(int pd, int gd, int od, int xd, const Launch& L, const mxopt_rmsprop_hp& hp,
                         const DevPrep& prep) {
  if (od != pd) return false;
  // as in launch_rmsprop: a lone 16-bit gradient with nothing in front of the square keeps its dtype there
  const int gsq_dtype = (L.npending == 0 && !prep_promotes(prep) && !hp.has_weight_decay) ? gd : MXOPT_F32;
  const RmspropMath math{hp, gsq_dtype};
  switch (pd) {
    case MXOPT_F32: return update_list_for_pd<MXOPT_F32>(gd, xd, L, math, prep);
    case MXOPT_BF16: return update_list_for_pd<MXOPT_BF16>(gd, xd, L, math, prep);
    case MXOPT_F16: return update_list_for_pd<MXOPT_F16>(gd, xd, L, math, prep);
  }
  return false;
}

}  // namespace mxopt
