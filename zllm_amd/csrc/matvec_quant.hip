// The decode multiply over quantized rows: which format's kernels (matvec_quant.h) a dispatch takes.
#include "matvec_quant.h"

namespace zhip {

zhip_result launch_matvec_quant(const Dispatch &d, const MvArgs &a, int type) {
    switch (type) {
    case 8: return launch_matvec_quant_q8(d, a);
    case 3: return launch_matvec_quant_q3(d, a);
    case 4: return launch_matvec_quant_q4(d, a);
    case 5: return launch_matvec_quant_q5(d, a);
    case 6: return launch_matvec_quant_q6(d, a);
    default: return fail(d, ZHIP_E_BAD_COMMAND, "decode multiply: no tuned kernel for type %d", type);
    }
}

}  // namespace zhip
