// Instantiates the K-source reduction for one (element type, fold) pair.
// Compiled once per pair with -DMDH_TNAME=<f32|f64|i32|i64|bf16|f16>
// -DMDH_FNAME=<sum|min|max>.
#include "reduce_kernels.h"

namespace mdh {
namespace {
using f32 = float;
using f64 = double;
using i32 = int32_t;
using i64 = int64_t;
using bf16 = bf16_t;
using f16 = f16_t;
[[maybe_unused]] constexpr int sum = kSum;
[[maybe_unused]] constexpr int min = kMin;
[[maybe_unused]] constexpr int max = kMax;
} // namespace

#define MDH_CAT2(a, b, c, d) a##b##c##d
#define MDH_CAT(a, b, c, d) MDH_CAT2(a, b, c, d)

int MDH_CAT(reduce_launch_, MDH_TNAME, _, MDH_FNAME)(const ReduceArgs& a, hipStream_t stream) {
  return launch<MDH_TNAME, MDH_FNAME>(a, stream);
}

int MDH_CAT(reduce_many_launch_, MDH_TNAME, _, MDH_FNAME)(const ManyJob* jobs, int njobs, int mode, float scale,
    bool spread, hipStream_t stream) {
  return launch_many<MDH_TNAME, MDH_FNAME>(jobs, njobs, mode, scale, spread, stream);
}
} // namespace mdh
