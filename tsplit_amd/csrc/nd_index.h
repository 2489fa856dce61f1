// Host-side description of an n-D strided walk, shared by the gather (broadcast / pad /
// transpose) and reduction kernels: a list of axes, outermost first, each with an extent and
// the element stride of the tensor being read; axes of extent 1 are dropped and neighbours
// that form one contiguous run are merged, so that the kernels see as few axes as possible.
#pragma once
#include <climits>
#include <cstdint>

#include "fastdiv.h"

namespace tsplit {

constexpr int kMaxDim = 8;

struct Axis {
  int64_t ext = 1;       // extent of the walk along this axis
  int64_t stride = 0;    // element stride in the tensor being read (0 = broadcast)
  int64_t lo = 0;        // read coordinate = walk coordinate - lo
  int64_t in_ext = -1;   // coordinates outside [0, in_ext) are not read; -1 = no limit
  int64_t stride2 = 0;   // element stride in a second tensor walked alongside (0 if unused)
  bool plain() const { return lo == 0 && (in_ext < 0 || in_ext >= ext); }
};

// Drops extent-1 axes and merges (outer, inner) pairs with outer.stride == inner.stride *
// inner.ext (and the same for stride2) when neither restricts its coordinates.  Returns the
// new count; at least one axis is always left.
inline int collapse_axes(Axis *a, int n) {
  int m = 0;
  for (int i = 0; i < n; ++i) {
    if (a[i].ext == 1 && a[i].plain()) continue;
    if (m > 0 && a[m - 1].plain() && a[i].plain() && a[m - 1].stride == a[i].stride * a[i].ext &&
        a[m - 1].stride2 == a[i].stride2 * a[i].ext) {
      a[m - 1].ext *= a[i].ext;
      a[m - 1].stride = a[i].stride;
      a[m - 1].stride2 = a[i].stride2;
      a[m - 1].in_ext = -1;
    } else {
      a[m++] = a[i];
    }
  }
  if (m == 0) {
    a[0] = Axis{};
    m = 1;
  }
  return m;
}

}  // namespace tsplit
