// gfx950 (CDNA4, MI355X) device code for allpaka's fused per-layer ops.
//
// Built with `hipcc --genco --offload-arch=gfx950 -ffp-contract=off` into one
// code object that the host library embeds and loads with hipModuleLoadData.
// Every kernel here is HBM-bound: wave64, 128-bit global accesses, DPP/shuffle
// reductions inside a wave, LDS only for cross-wave sums and byte staging.
// No MFMA: nothing on this path is a contraction.
//
// Arithmetic contract (what the CPU reference computes, op for op):
//   * -ffp-contract=off for the whole file: a*b-c stays two rounded f32 ops,
//     as in the reference's Rust (dequant.rs:221-228, rope.rs:75-80).
//   * RMS statistics are accumulated and applied in f64 (norm.rs:115-187):
//     out = ((x as f64 * scale) as f32) * w.
//   * fp16 activations (a storage form the reference does not have) are
//     widened to f32 on load and rounded once (RNE) on store.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kernels/common.hip.h"
#include "kernels/elementwise.hip.h"
#include "kernels/addnorm.hip.h"
#include "kernels/combine.hip.h"
#include "kernels/argmax.hip.h"
#include "kernels/qknorm_rope.hip.h"
#include "kernels/embed.hip.h"
#include "kernels/router.hip.h"
#include "kernels/permute.hip.h"
