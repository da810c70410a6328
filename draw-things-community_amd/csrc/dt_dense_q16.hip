// K1 instantiations for plain fp16 weights (all tile shapes, with and without the elementwise tail).
#include "dt_dense_launch.h"

namespace dt {
template dt_status launch_dense_q<16>(hipStream_t, const DenseArgs&, int, bool, int);
}  // namespace dt
