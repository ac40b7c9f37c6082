// Knobs of the `hip` dialect that have no field in the reference's schemas.
#pragma once

namespace raf {
namespace op {
namespace hip {

// Factor every LANS gradient is multiplied by before use (undoing a loss scale, e.g. 1/1024 for
// fp16 gradients).  Captured when a LANS OpEnv is made; 1 by default.  The reference's LansArgs
// has no such field: there, gradients are cast and unscaled by separate ops before LANS runs.
void SetLansGradUnscale(float factor);
float GetLansGradUnscale();

}  // namespace hip
}  // namespace op
}  // namespace raf
