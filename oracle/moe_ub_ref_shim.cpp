// C entry points over the reference's own header include/catccos/detail/ascend950_moe_ub.h, compiled
// only where the reference checkout is present (see Makefile).  Lets a test compare the oracle's
// restated sizing formulas with the reference's code on arbitrary arguments.  Test infrastructure.
#include "catccos/detail/ascend950_moe_ub.h"

using Ub = Catccos::Detail::Ascend950MoeUb;

extern "C" {
unsigned long long ref_ub_input_quant_bytes(unsigned hidden) { return Ub::InputQuantBytes(hidden); }
unsigned long long ref_ub_dispatch_bytes(unsigned hidden) { return Ub::DispatchBytes(hidden); }
unsigned long long ref_ub_unpermute_bytes(unsigned m, unsigned hidden, unsigned topk, unsigned aiv) {
    return Ub::UnpermuteBytes(m, hidden, topk, aiv);
}
int ref_ub_fits(unsigned m, unsigned hidden, unsigned topk, unsigned aiv) { return Ub::Fits(m, hidden, topk, aiv) ? 1 : 0; }
}
