// Entry points of the decode-step glue kernels (RMSNorm, RoPE, embedding,
// residual add, LM-head argmax).
#include "kernels/kernels.h"
#include "runtime.h"

namespace llmopt {

void register_glue_kernels(std::vector<KernelEntryPoint> &table) { (void)table; }

}  // namespace llmopt
