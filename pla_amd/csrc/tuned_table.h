// Tuned rows-per-wavefront table of the k-last decode kernels.
//
// The table text is generated from the auto-tuner's result files (pla_amd/lut/*.csv) on every build; the
// reference generates its dispatch from the same kind of file
// (scripts/decode/generate_kernel_instantiations.py, lut/tuned_result_<device>.csv).  A shape that the
// table holds takes the row count tuned at the nearest batch size (in ratio); every other shape falls
// back to the size thresholds of the caller.
#pragma once

namespace pla {

enum TunedKernel { TUNED_K_LAST = 0, TUNED_K_LAST_PACKED = 1, TUNED_K_LAST_MTP = 2 };

struct TunedRow { int kernel, tree, act_dtype, state_dtype, H, HV, B, rows_per_wave; };

#include "generated/tuned_table.inc"

// 0 if the shape is not in the table.  The rows are sorted by (kernel, tree, dtypes, H, HV, B): the rows of a shape
// are found by bisection (the lookup is on the launch path of every decode call), then scanned for the batch size
// that is nearest in ratio.
static int tuned_rows_per_wave(const TunedRow* rows, int count, int kernel, int tree, int act_dtype,
                               int state_dtype, int H, int HV, int B) {
  const int want[6] = {kernel, tree, act_dtype, state_dtype, H, HV};
  auto shape_less = [&](const TunedRow& r) {          // r's shape sorts before the wanted one
    const int have[6] = {r.kernel, r.tree, r.act_dtype, r.state_dtype, r.H, r.HV};
    for (int i = 0; i < 6; ++i)
      if (have[i] != want[i]) return have[i] < want[i];
    return false;
  };
  int lo = 0, hi = count;
  while (lo < hi) {
    const int mid = (lo + hi) / 2;
    if (shape_less(rows[mid])) lo = mid + 1; else hi = mid;
  }
  int best = 0;
  double best_ratio = 0.0;
  for (int i = lo; i < count; ++i) {
    const TunedRow& r = rows[i];
    if (r.kernel != kernel || r.tree != tree || r.act_dtype != act_dtype || r.state_dtype != state_dtype ||
        r.H != H || r.HV != HV)
      break;
    if (r.B <= 0) continue;
    const double ratio = r.B > B ? (double)r.B / B : (double)B / r.B;
    if (best == 0 || ratio < best_ratio) { best = r.rows_per_wave; best_ratio = ratio; }
  }
  return best;
}

}  // namespace pla
