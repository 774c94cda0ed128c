// Test infrastructure only. Python entry point for a CPU-only build of four of
// the reference's own translation units (ops/timestep_norm.cc,
// ops/ema_parameters.cc, ops/ema_hidden.cc, ops/sequence_norm.cc), compiled where they lie under
// /root/reference by oracle/Makefile. Nothing of the reference is copied: this
// file only registers the op tables those translation units already define.
// The CUDA entry points they dispatch to stay unresolved (lazy binding); they
// are never reached for CPU tensors.
#include <torch/extension.h>

#include "ops/ema_hidden.h"
#include "ops/ema_parameters.h"
#include "ops/sequence_norm.h"
#include "ops/timestep_norm.h"

PYBIND11_MODULE(mega2_ref_cpu, m) {
  m.doc() = "CPU translation units of the reference, for oracle validation";
  mega2::ops::DefineTimestepNormOp(m);
  mega2::ops::DefineEMAParametersOp(m);
  mega2::ops::DefineEMAHiddenOp(m);
  mega2::ops::DefineSequenceNormOp(m);
}
