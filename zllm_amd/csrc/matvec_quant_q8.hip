// matvec_q8_0: the default decode kernels of matvec_quant.h for this format.
#include "matvec_quant.h"

namespace zhip {

zhip_result launch_matvec_quant_q8(const Dispatch &d, const MvArgs &a) { return launch_quant<KQ8>(d, a); }

}  // namespace zhip
