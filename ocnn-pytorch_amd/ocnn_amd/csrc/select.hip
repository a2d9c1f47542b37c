// Which kernel runs a layer: the selection among the gather-GEMM and weight-gradient entry
// points, as one pair of functions of the C ABI, so that whoever binds the header gets the
// same choices as the Python layer of this package (which calls these functions too).
//
// Every *_supported() predicate says whether a kernel takes a shape class; the row ranges that
// its entry point checks on top (32-bit buffer offsets of the output, of the table, of the
// plan) are repeated here, so a choice is always one that the chosen entry point accepts.
#include "common.hpp"

using namespace ocnn;

namespace {

constexpr int64_t kOffsetLimit = 0xfff00000ll;   // what a 32-bit buffer offset may reach
constexpr int kPadMinRows = 16384;               // from here on odd channel counts run zero-padded
constexpr double kSparseMaxOccupancy = 0.3;      // share of table entries set, up to which the pair plan pays
constexpr int64_t kSparseMinRows = 32768;        // (its workgroups load their weights once per launch)

bool rows_ok(int64_t rows_out, int64_t plan_total) {
  return rows_out >= 0 && rows_out < (1ll << 31) && plan_total >= 0 && plan_total < (1ll << 29);
}

}  // namespace

extern "C" int ocnn_conv_gather_choose(int dtype, int64_t rows_in, int64_t rows_out, int K, int cin, int cout,
                                       int identity_table, int has_plan, int plan_max_distinct,
                                       int64_t plan_total, double plan_occupancy, double plan_reuse) {
  const bool known = dtype == OCNN_F32 || dtype == OCNN_F16 || dtype == OCNN_BF16;
  if (rows_out >= kPadMinRows && known && (cin % 32 != 0 || cout % 16 != 0)) return OCNN_GATHER_ZERO_PADDED;
  if (identity_table && K == 1 && rows_out == rows_in) {
    if (ocnn_conv_dense_rw_supported(dtype, rows_out, cin, cout)) return OCNN_GATHER_DENSE_RW;
    // (many input channels into few output channels: the row tile that fits LDS is small and
    // the weights are streamed once per tile; the plan-free kernel is no slower there)
    if (!(cin >= 512 && cout < 256) && ocnn_conv_dense_supported(dtype, rows_out, cin, cout))
      return OCNN_GATHER_DENSE;
  }
  if (has_plan && rows_ok(rows_out, plan_total)) {
    if (ocnn_conv_gather_rw_supported(dtype, rows_in, K, cin, cout, plan_max_distinct) &&
        rows_out * K * 2 < kOffsetLimit && (rows_out + 128) * cout * 2 < kOffsetLimit)
      return OCNN_GATHER_RW;
    // (eight slots - the 2x2x2 tables and their inverses - stream a third of the weights of 27 per
    // tile: there the kernel for wide layers beats the pair plan also at one slot in eight set,
    // 0.84 -> 0.67 ms for 96 -> 96 between depths 9 and 8, and without rows shared inside a tile)
    if (K == 8 && ocnn_conv_gather_wide_supported(dtype, rows_in, K, cin, cout, plan_max_distinct))
      return OCNN_GATHER_WIDE;
    if (plan_occupancy <= kSparseMaxOccupancy && rows_out >= kSparseMinRows &&
        rows_out * cout * 2 <= kOffsetLimit &&
        ocnn_conv_gather_sparse_supported(dtype, rows_in, K, cin, cout, plan_max_distinct))
      return OCNN_GATHER_SPARSE;
    // (staging a tile's distinct rows pays when rows are used more than once per tile)
    if (plan_reuse >= 2.0 && ocnn_conv_gather_wide_supported(dtype, rows_in, K, cin, cout, plan_max_distinct))
      return OCNN_GATHER_WIDE;
    if (plan_reuse >= 2.0 && K <= 27 && ocnn_conv_gather_planned_supported(dtype, rows_in, cin, cout))
      return OCNN_GATHER_PLANNED;
  }
  return OCNN_GATHER_PLAIN;
}

extern "C" int ocnn_conv_wgrad_choose(int dtype, int64_t rows_x, int64_t rows, int K, int ca, int cb,
                                      int identity_table, int has_plan, int plan_max_distinct,
                                      int64_t plan_total, double plan_occupancy) {
  const bool known = dtype == OCNN_F32 || dtype == OCNN_F16 || dtype == OCNN_BF16;
  if (rows >= kPadMinRows && known && (ca % 32 != 0 || cb % 32 != 0)) return OCNN_WGRAD_ZERO_PADDED;
  // (below some 8 k channel pairs a workgroup's 128 k-pair block is mostly zeros and the
  // plan-free kernel is as fast)
  if (identity_table && K == 1 && rows_x == rows && (int64_t)ca * cb >= 8192 &&
      ocnn_conv_dense_wgrad_rw_supported(dtype, rows, ca, cb))
    return OCNN_WGRAD_DENSE_RW;
  if (has_plan && rows_ok(rows, plan_total) && rows * K * 2 < kOffsetLimit) {
    // (32 x 32 and 64 x 64 have planned kernels of their own that are faster still; with channel
    // counts that are not multiples of 64 on the table-row side the pair-plan kernel, which sums
    // exactly ca x cb and only over the pairs, beats zero-padded 64 x 64 blocks on dense tables too)
    if ((plan_occupancy <= kSparseMaxOccupancy || cb % 64 != 0) && rows >= kSparseMinRows &&
        !(ca == cb && (ca == 32 || ca == 64)) &&
        ocnn_conv_wgrad_sparse_supported(dtype, rows_x, rows, K, ca, cb, plan_max_distinct))
      return OCNN_WGRAD_SPARSE;
    if (ocnn_conv_wgrad_planned_supported(dtype, rows_x, rows, K, ca, cb, plan_max_distinct))
      return OCNN_WGRAD_PLANNED;
  }
  return OCNN_WGRAD_PLAIN;
}
