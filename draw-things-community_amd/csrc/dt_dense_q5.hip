// K1 instantiations for 5-bit palette indices (all tile shapes, with and without the elementwise tail).
#include "dt_dense_launch.h"

namespace dt {
template dt_status launch_dense_q<5>(hipStream_t, const DenseArgs&, int, bool, int);
}  // namespace dt
