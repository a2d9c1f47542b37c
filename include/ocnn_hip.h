/*
 * ocnn_hip.h - C ABI of the MI355X (gfx950) octree sparse-convolution library.
 *
 * The reference (octree-nn/ocnn-pytorch) has no FFI: its hot path is Python
 * calling torch ops and Triton kernels.  Each entry point below names the
 * reference code it stands in for (paths relative to the reference checkout).
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless its name starts with "h_";
 *   - `stream` is a hipStream_t passed as void*; work is enqueued, not awaited;
 *   - the library never allocates device memory: outputs and workspaces are
 *     supplied by the caller (sizes from the *_workspace_bytes queries);
 *   - return value 0 = ok, negative = error (text from ocnn_last_error());
 *   - arguments are checked on the host before anything is launched: a NULL in place of an
 *     array that the call reads or writes (with the sizes given; an operand of zero rows may
 *     be NULL), a negative size or an unsupported shape is OCNN_ERR_ARG, a workspace that is
 *     too small OCNN_ERR_WORKSPACE; pointers named "may be NULL" are optional;
 *   - feature matrices are row-major (rows, channels); neighbour tables are
 *     row-major (rows, K) int32 with -1 for "no neighbour";
 *   - dtype codes: 0 = float32, 1 = float16, 2 = bfloat16 (fp32 accumulation);
 *   - sizes the reference does not limit and this library does (OCNN_ERR_ARG beyond them):
 *     a neighbour table has fewer than 2^31 entries (79.5 M rows of 27 slots), a layer
 *     and a point cloud fewer than 2^31 nodes / points, full layers reach depth 8 in the
 *     build and depth 7 in the neighbour search (batch x 8^depth x 27 < 2^31), octrees
 *     depth 16 (what 48-bit keys hold); the kernels on a tile plan address their tensors
 *     with 32-bit byte offsets (rows x channels x 2 bytes below 0xfff00000: their
 *     ..._supported() and the ..._choose() functions tell, and the plan-free entry points
 *     take what is larger).
 */
#ifndef OCNN_HIP_H_
#define OCNN_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define OCNN_F32 0
#define OCNN_F16 1
#define OCNN_BF16 2

#define OCNN_OK 0
#define OCNN_ERR_ARG (-1)      /* bad argument / unsupported shape          */
#define OCNN_ERR_HIP (-2)      /* a HIP call or launch failed               */
#define OCNN_ERR_WORKSPACE (-3)/* workspace too small                       */

const char* ocnn_last_error(void);
int ocnn_abi_version(void);

/* ---- Morton keys ------------------------------------------------------- */

/* ocnn/octree/shuffled_key.py:60-90 (xyz2key).  b may be NULL. */
int ocnn_xyz2key(const int64_t* x, const int64_t* y, const int64_t* z,
                 const int64_t* b, int64_t n, int depth, int64_t* key,
                 void* stream);

/* ocnn/octree/shuffled_key.py:93-115 (key2xyz). */
int ocnn_key2xyz(const int64_t* key, int64_t n, int depth, int64_t* x,
                 int64_t* y, int64_t* z, int64_t* b, void* stream);

/* ocnn/octree/points.py:223-244 (Points.normalize) fused with the key
 * computation of ocnn/octree/octree.py:219-226: pts_out = (pts - bbmin) *
 * factor in fp32 (no FMA contraction), key = xyz2key(trunc(pts_out), batch).
 * batch (one id per point) may be NULL; batch_is_float selects float32 ids
 * (as Points.merge_points makes them) or int64 ids.  h_bbmin: 3 host floats. */
int ocnn_points2key(const float* pts, int64_t n, const float* h_bbmin,
                    float factor, const void* batch, int batch_is_float,
                    int depth, float* pts_out, int64_t* key, void* stream);

/* Host-side evaluation of the bit arithmetic the two kernels above use, so
 * that it can be checked without a GPU.  xyzb: 4 host int64. */
int64_t ocnn_host_encode_key(int64_t x, int64_t y, int64_t z, int64_t b, int depth);
void ocnn_host_decode_key(int64_t key, int depth, int64_t* h_xyzb);

/* ---- octree build ------------------------------------------------------ */

/* The whole of ocnn/octree/octree.py:227-270 above the point keys
 * (torch.unique with inverse, then one unique_consecutive per layer) in two
 * calls with ONE read-back between them (the reference reads a count back per
 * layer).
 * scan: sorts the n keys (batch id packed above the 3 * depth Morton bits;
 *       batch_bits = bits of the largest batch id), perm[n] = the stable
 *       sorting order, and numbers the nodes of every layer in one scan.
 *       sizes (device, depth - full_depth + 1 values): sizes[0] = leaves,
 *       sizes[l] = non-empty nodes l layers above them.
 * fill: h_sizes = sizes read back (host).  h_keys / h_children: host arrays of
 *       depth + 1 device pointers, layer d holding batch_size * 8^d nodes for
 *       d <= full_depth and 8 * h_sizes[depth - d + 1] below.  Writes every
 *       layer's keys and children, inverse[n] (point -> leaf, the reference's
 *       idx) and seg_start[sizes[0] + 1] (leaf -> its run in perm).  Same
 *       workspace as given to scan, untouched in between. */
int64_t ocnn_octree_build_workspace_bytes(int64_t n, int depth, int full_depth,
                                          int batch_bits);
int ocnn_octree_build_scan(const int64_t* key, int64_t n, int depth,
                           int full_depth, int batch_bits, void* workspace,
                           int64_t workspace_bytes, int32_t* perm,
                           int64_t* sizes, void* stream);
int ocnn_octree_build_fill(const void* workspace, int64_t n, int depth,
                           int full_depth, int batch_size, int batch_bits,
                           const int64_t* h_sizes, const int32_t* perm,
                           int64_t* const* h_keys, int32_t* const* h_children,
                           int64_t* inverse, int32_t* seg_start, void* stream);

/* A full layer (ocnn/octree/octree.py:289-321): keys[i] = (i mod 8^depth) |
 * (i div 8^depth) << 48 for the batch_size * 8^depth nodes; children[i] = i
 * when with_children != 0, else -1. */
int ocnn_build_full_layer(int depth, int batch_size, int with_children,
                          int64_t* keys, int32_t* children, void* stream);


/* Regrowing an octree from split decisions, ocnn/octree/octree.py:323-351 (octree_split) and
 * :353-402 (octree_grow).
 * split_children: children[i] = ordinal of node i among the nodes with split[i] != 0, or -1;
 *        *count (device) = their number.  A layer without any split node keeps node 0
 *        (children[0] = 0, count 1), as the reference does.  Workspace:
 *        ocnn_build_level_workspace_bytes(n) bytes.
 * grow_layer: the layer below `n_nempty` non-empty nodes (nempty_index = their rows, keys of
 *        their layer in key_above): keys[8 p + j] = key of the p-th of them with j appended
 *        below the batch bits, children[8 p + j] = 8 p + j. */
int64_t ocnn_build_level_workspace_bytes(int64_t n);
int ocnn_split_children(const int32_t* split, int64_t n, void* workspace, int64_t workspace_bytes,
                        int32_t* children, int64_t* count, void* stream);
int ocnn_grow_layer(const int64_t* key_above, const int32_t* nempty_index, int64_t n_nempty,
                    int64_t* keys, int32_t* children, void* stream);

/* Per-leaf signal of ocnn/octree/octree.py:273-281: sequential fp32 sum of
 * the leaf's points (in point order), then mode 0: divide by the count
 * (points, features); mode 1: L2-normalise with eps 1e-12 (normals). */
int ocnn_leaf_average(const float* src, int channels, const int32_t* perm,
                      const int32_t* seg_start, int64_t n_leaf, int mode,
                      float* out, void* stream);
/* The two calls a cloud with normals needs (mode 0 on the scaled points, mode 1 on the normals,
 * 3 channels each) in one pass over the leaves' points; same sums, same results. */
int ocnn_leaf_points_normals(const float* pts, const float* normals, const int32_t* perm,
                             const int32_t* seg_start, int64_t n_leaf, float* out_pts,
                             float* out_normals, void* stream);

/* ---- neighbour search -------------------------------------------------- */

/* ocnn/octree/octree.py:411-428: 27-neighbour table of a full layer,
 * (batch * 8^depth, 27).  out64 or out32 may be NULL. */
int ocnn_neigh_full(int depth, int batch, int64_t* out64, int32_t* out32,
                    void* stream);

/* ocnn/octree/octree.py:430-439: table of depth d from the table of depth
 * d-1.  child_p: children[d-1] (n_p nodes); neigh_p: (n_p, 27) table of depth
 * d-1; nempty_p: node index of each of the n_ne non-empty parents in order.
 * Output rows 8c..8c+7 belong to parent ordinal c: (8*n_ne, 27). */
int ocnn_neigh_from_parent(const int32_t* child_p, const int32_t* neigh_p,
                           const int32_t* nempty_p, int64_t n_ne,
                           int64_t* out64, int32_t* out32, void* stream);

/* construct_all_neigh (ocnn/octree/octree.py:443-446) as one call: layers 1 .. depth in turn,
 * ocnn_neigh_full up to full_depth, then ocnn_nempty_index of the layer above (written to
 * h_nempty_index[d - 1], int32) and ocnn_neigh_from_parent.  h_*: host arrays indexed by depth
 * (depth + 1 entries; node counts, children, outputs); tables int32 (nnum[d], 27). */
int ocnn_neigh_all(int depth, int full_depth, int batch, const int64_t* h_nnum,
                   const int64_t* h_nnum_nempty, const int32_t* const* h_children,
                   int32_t* const* h_nempty_index, int32_t* const* h_neigh, void* stream);

/* Host evaluation of the arithmetic that replaces the reference's lut_parent /
 * lut_child tables (ocnn/octree/octree.py:87-95) inside the kernel above. */
void ocnn_host_child_slot_lut(int j, int k, int* lut_parent, int* lut_child);

/* ocnn/octree/octree.py:160-172 (nempty_index): index[children[q]] = q for
 * children[q] >= 0.  index32 / index64 may be NULL. */
int ocnn_nempty_index(const int32_t* children, int64_t n, int32_t* index32,
                      int64_t* index64, void* stream);

/* ocnn/octree/octree.py:188-199 and :490-523 (remap_nempty_neigh, get_neigh)
 * in one pass: out[i][c] = remap(neigh[row(i)][cols[c]]) with
 * row(i) = row_index[i] if row_index else i * row_stride, and
 * remap(v) = v < 0 ? -1 : (children ? children[v] : v).
 * h_cols: K host ints (column selection, NULL = identity over 27). */
int ocnn_neigh_select(const int32_t* neigh, const int32_t* row_index,
                      int row_stride, const int32_t* children,
                      const int* h_cols, int K, int64_t rows, int64_t* out64,
                      int32_t* out32, void* stream);

/* Widening copy of a table (the public int64 view of an int32 table). */
int ocnn_table_to_i64(const int32_t* in, int64_t n, int64_t* out, void* stream);
int ocnn_table_to_i32(const int64_t* in, int64_t n, int32_t* out, void* stream);

/* Inverse of a table: out (rows_in, K) with out[t[i][k]][k] = i, -1 elsewhere.
 * Valid because every (input row, slot) has at most one producer.  Turns the
 * scatter of ocnn/nn/octree_conv.py:160-166 (backward_gemm) into a gather. */
int ocnn_table_transpose(const int32_t* table, int64_t rows, int K,
                         int64_t rows_in, int32_t* out, void* stream);

/* ---- convolution engine ------------------------------------------------ */

/* Gather-GEMM: out[i][:] = sum_k [t[i][k] >= 0] in[t[i][k]][:] @ Wk (+ bias)
 * where Wk = w[k'] (cin, cout) or its transpose, k' = k or K-1-k.
 *   w_transposed = 0: w is (K, cin, cout)      (forward_gemm,
 *                     ocnn/nn/octree_conv.py:115-143)
 *   w_transposed = 1: w is (K, cout, cin)      (backward_gemm :145-168 in
 *                     gather form; reverse_slots = 1 uses the mirrored slot of
 *                     a centrally symmetric table instead of a transposed one,
 *                     as ocnn/nn/kernels/conv_bwd_implicit_gemm.py:56 does)
 * bias may be NULL.  Rows of `in` are addressed by table values only.
 * workspace: ocnn_conv_workspace_bytes(K, cin, cout) bytes (packed weights). */
int64_t ocnn_conv_workspace_bytes(int K, int cin, int cout);
/* Workspace of ocnn_conv_gather including, for fp32 with cin % 32 == 0 and cout % 16 == 0,
 * the room to run on the bf16 MFMA kernel as three bf16 pieces ([hi | hi | lo] input channels
 * against [hi; lo; hi] weights, fp32 accumulation and output, about 1e-5 relative).  With
 * only ocnn_conv_workspace_bytes() of room fp32 runs on the plain kernel. */
int64_t ocnn_conv_gather_workspace_bytes(int dtype, int64_t rows_in, int K, int cin, int cout);
int ocnn_conv_gather(int dtype, const void* in, int64_t rows_in,
                     const int32_t* table, int64_t rows_out, int K,
                     const void* w, int cin, int cout, int w_transposed,
                     int reverse_slots, const void* bias, void* out,
                     void* workspace, int64_t workspace_bytes, void* stream);

/* Tile plan of a table: for every tile of ocnn_tile_plan_rows() consecutive
 * table rows, the ascending list of distinct rows the tile reads, and for every
 * table entry its position in that list plus one (0 for -1).  Lets a kernel bring
 * each distinct row into LDS once per tile instead of once per (row, slot).
 *   count: ucount[tile] = number of distinct rows        (tiles = ceil(rows / R));
 *          tile_nnz[tile] (may be NULL) = entries of the tile that hold a row;
 *   offsets: uptr (tiles + 1) = exclusive prefix sum of ucount, and what the host needs to
 *          size the lists, stats (device, 6 x int64) = [tiles with more than cap distinct
 *          rows, dropped (0 | 1), total, largest count, entries set, tiles the one-pass
 *          build gave up on].  When the tiles over cap are few (at most a tenth of the
 *          tiles, at least one) they are dropped: they count as empty in uptr and in the
 *          third to fifth figure, and the caller runs their rows without the plan;
 *   fill : uptr as made by offsets (or by the caller);
 *          urows[uptr[tile] + u] = u-th distinct row; loc (tiles, K, R) uint16:
 *          loc[tile][k][r] = 1 + position of table[tile * R + r][k], or 0 for -1 and
 *          for the rows of the last tile past the table.
 * No counterpart in the reference: its kernels gather per (row, slot)
 * (ocnn/nn/kernels/conv_fwd_implicit_gemm.py:57-72). */
int ocnn_tile_plan_rows(void);
int ocnn_tile_plan_count(const int32_t* table, int64_t rows, int K, int32_t* ucount,
                         int32_t* tile_nnz, void* stream);
int ocnn_tile_plan_offsets(const int32_t* ucount, const int32_t* tile_nnz, int64_t tiles, int cap,
                           int32_t* uptr, int64_t* stats, void* stream);
int ocnn_tile_plan_fill(const int32_t* table, int64_t rows, int K, const int32_t* uptr,
                        int32_t* urows, uint16_t* loc, void* stream);
/* The same plan with ONE pass over the table instead of two: ocnn_tile_plan_build counts
 * (as ocnn_tile_plan_count) and writes the positions and, at the fixed place
 * ulist[tile * pad + u], the lists of the tiles with at most `pad` distinct rows;
 * ocnn_tile_plan_offsets as above; ocnn_tile_plan_compact moves the lists to their offsets
 * and clears the positions of the tiles the offsets dropped (stats: the device vector that
 * ocnn_tile_plan_offsets wrote; cap <= pad).  A plan whose largest count (stats[3]) exceeds
 * `pad` is filled with ocnn_tile_plan_fill instead.  The build keeps a tile's distinct rows
 * in a small set (1024 blocks of 32 row numbers; the tiles of an octree table use a tenth),
 * so that four tiles share a CU: a tile that does not fit gets the count 2^20 and is counted
 * in stats[5]; such a table (one without locality) is planned with count, offsets and fill. */
int ocnn_tile_plan_build(const int32_t* table, int64_t rows, int K, int pad, int32_t* ucount,
                         int32_t* tile_nnz, int32_t* ulist, uint16_t* loc, void* stream);
int ocnn_tile_plan_compact(const int32_t* ucount, const int32_t* uptr, const int64_t* stats, int cap,
                           int pad, const int32_t* ulist, int32_t* urows, uint16_t* loc, int K,
                           int64_t tiles, void* stream);

/* ---- kernel selection ----------------------------------------------------
 * Which entry point runs a gather-GEMM (forward_gemm / backward_gemm in gather form,
 * ocnn/nn/octree_conv.py:115-168) or a weight gradient (weight_gemm, :170-202) of a given
 * shape: the reference picks between its Triton and torch paths in Python
 * (ocnn/nn/octree_conv.py:347-357); here the choice among the kernels is part of the ABI.
 * A returned code names an entry point that accepts the shape (its *_supported() predicate
 * and the row ranges it checks).  identity_table: the table is the one-slot identity (row i
 * reads row i: the dense form of 2x2x2 stride-2 layers and 1x1 convolutions).  Without a tile
 * plan pass has_plan = 0 (the other plan arguments are then ignored); plan_occupancy = share
 * of the table entries that are set, plan_reuse = entries set / distinct rows summed over
 * the tiles.  ZERO_PADDED: pad the channels with zeros to multiples of 32 (cout of a gather:
 * 16) and choose again. */
#define OCNN_GATHER_PLAIN 0        /* ocnn_conv_gather            */
#define OCNN_GATHER_DENSE_RW 1     /* ocnn_conv_dense_rw          */
#define OCNN_GATHER_DENSE 2        /* ocnn_conv_dense             */
#define OCNN_GATHER_RW 3           /* ocnn_conv_gather_rw         */
#define OCNN_GATHER_SPARSE 4       /* ocnn_conv_gather_sparse     */
#define OCNN_GATHER_WIDE 5         /* ocnn_conv_gather_wide       */
#define OCNN_GATHER_PLANNED 6      /* ocnn_conv_gather_planned    */
#define OCNN_GATHER_ZERO_PADDED 7
#define OCNN_WGRAD_PLAIN 0         /* ocnn_conv_wgrad             */
#define OCNN_WGRAD_DENSE_RW 1      /* ocnn_conv_dense_wgrad_rw    */
#define OCNN_WGRAD_SPARSE 2        /* ocnn_conv_wgrad_sparse      */
#define OCNN_WGRAD_PLANNED 3       /* ocnn_conv_wgrad_planned     */
#define OCNN_WGRAD_ZERO_PADDED 4
int ocnn_conv_gather_choose(int dtype, int64_t rows_in, int64_t rows_out, int K, int cin, int cout,
                            int identity_table, int has_plan, int plan_max_distinct,
                            int64_t plan_total, double plan_occupancy, double plan_reuse);
int ocnn_conv_wgrad_choose(int dtype, int64_t rows_x, int64_t rows, int K, int ca, int cb,
                           int identity_table, int has_plan, int plan_max_distinct,
                           int64_t plan_total, double plan_occupancy);

/* ocnn_conv_gather over a tile plan (same arguments otherwise, same result).
 * Supported for f16 / bf16 with cin and cout multiples of 64 and an input
 * smaller than 4 GiB; ocnn_conv_gather_planned_supported() tells. */
int ocnn_conv_gather_planned_supported(int dtype, int64_t rows_in, int cin, int cout);
int ocnn_conv_gather_planned(int dtype, const void* in, int64_t rows_in,
                             const uint16_t* loc, const int32_t* uptr,
                             const int32_t* urows, int64_t rows_out, int K,
                             const void* w, int cin, int cout, int w_transposed,
                             int reverse_slots, const void* bias, void* out,
                             void* workspace, int64_t workspace_bytes, void* stream);

/* ocnn_conv_gather for 64 -> 64 and 32 -> 32 channels with register-resident
 * weights: one persistent workgroup per CU keeps all K x C x C weights in VGPRs
 * (split over its four waves at C = 64, whole in every wave at C = 32) and walks
 * its tiles of the plan.  plan_max_distinct = largest number of distinct rows
 * of any tile (max of ucount); the kernel needs it <= 416.  plan_total = number
 * of entries of urows (uptr[tiles]).  Same result as ocnn_conv_gather. */
int ocnn_conv_gather_rw_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                  int plan_max_distinct);
int ocnn_conv_gather_rw(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                        const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                        int64_t plan_total, int64_t rows_out, int K, const void* w, int cin, int cout,
                        int w_transposed, int reverse_slots, const void* bias, void* out,
                        void* workspace, int64_t workspace_bytes, void* stream);

/* ocnn_conv_gather_rw without a workspace argument and without any allocation.  No
 * counterpart in the reference: it is for callers that cannot allocate device memory
 * (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  The
 * packed weights go to a device array built into the library, K * cin * cout * 2 bytes of
 * it, at most ocnn_conv_gather_rw_static_max_weight_bytes() = 221 184 (27 x 64 x 64); a
 * larger layer is rejected with OCNN_ERR_ARG.  Every GPU the library runs on holds its own
 * copy of the array until the process ends; all calls on one GPU share it, so calls that
 * overlap on one GPU (different streams or threads) race.  Same arguments otherwise, same
 * result bit for bit as ocnn_conv_gather_rw. */
int64_t ocnn_conv_gather_rw_static_max_weight_bytes(void);
int ocnn_conv_gather_rw_static(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                               const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                               int64_t plan_total, int64_t rows_out, int K, const void* w, int cin,
                               int cout, int w_transposed, int reverse_slots, const void* bias,
                               void* out, void* stream);

/* ocnn_conv_gather for wide layers (cin >= 64 and cout >= 96, multiples of 32, any
 * K <= 27) over the tile plan: the distinct rows of a tile are staged in LDS 64 input
 * channels at a time, the weights stream from L2 into registers in the MFMA operand
 * layout, the four waves of a workgroup split the output channels.  Same arguments and
 * result as ocnn_conv_gather_rw; plan_max_distinct <= 416; workspace K * cin64 * cout * 2 bytes
 * with cin64 = cin rounded up to a multiple of 64.  plan_occupancy: the share of the table's
 * entries that are set (as for ocnn_conv_gather_choose), negative if unknown: from 40 % down
 * (other than 2x2x2 tables) the kernel tests, per slot and 32-row block of a tile, whether any
 * row has an entry there and leaves the block's products out otherwise: the rows of empty
 * entries are zeros (as in the reference's buffer, ocnn/nn/octree_conv.py:133-137), so the
 * result is the same. */
int ocnn_conv_gather_wide_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                    int plan_max_distinct);
int ocnn_conv_gather_wide(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                          const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                          int64_t plan_total, double plan_occupancy, int64_t rows_out, int K,
                          const void* w, int cin, int cout, int w_transposed, int reverse_slots,
                          const void* bias, void* out, void* workspace, int64_t workspace_bytes,
                          void* stream);

/* Pair plan of a table, on top of its tile plan (loc: tiles x K x ocnn_tile_plan_rows()):
 * what ocnn_conv_gather_sparse and ocnn_conv_wgrad_sparse walk over.  It holds, per tile and
 * LIST, the rows that have a neighbour, in blocks of 16 pairs.  A list is a slot of the
 * table, or - for a slot with many pairs, like the centre of a 3x3x3 table - the rows
 * r0 .. r1 - 1 of the tiles of that slot: list = slot | r0 << 8 | (r1 - 1) << 16.  No
 * counterpart in the reference.
 *   slot_counts: slot_count[k] (device, K x int64) = table entries of slot k that hold a row;
 *   lists (host only, host arrays): cuts heavy slots by rows, deals the lists (at most 32)
 *          to four groups of at most 8 with about equal numbers of pairs; lists in group
 *          order, list_count[j] = pairs of list j (estimated for cut slots), group g = lists
 *          group_bounds[g] .. group_bounds[g + 1] - 1;
 *   count: nblk[tile * n_lists + j] = blocks of 16 pairs of list j in the tile (lists: a
 *          device copy of the array);
 *   fill : cptr (tiles * n_lists + 1) = exclusive prefix sum of nblk, made by the caller;
 *          ent (16 entries per block): position of the pair's input row in the tile's list
 *          of rows + 1, | r << 16 for row r of the tile; the last block
 *          of a list is filled up with position 0, r = 128. */
int ocnn_pair_plan_slot_counts(const uint16_t* loc, int64_t tiles, int K, int64_t* slot_count,
                               void* stream);
int ocnn_pair_plan_lists(int K, const int64_t* slot_count, int32_t* lists, int64_t* list_count,
                         int32_t* group_bounds, int* n_lists);
int ocnn_pair_plan_count(const uint16_t* loc, int64_t tiles, int K, const int32_t* lists,
                         int n_lists, int32_t* nblk, void* stream);
int ocnn_pair_plan_fill(const uint16_t* loc, int64_t tiles, int K, const int32_t* lists,
                        int n_lists, const int32_t* cptr, uint32_t* ent, void* stream);

/* ocnn_conv_gather for sparse tables (few of the K slots of a row hold a neighbour, as on the
 * non-empty nodes of a deep level): the work follows the (row, neighbour) pairs.  On top of
 * the tile plan (uptr, urows) it takes the pair plan of the table (cptr, ent, n_blocks = all
 * blocks, max_blocks = the most blocks of one tile, lists as a device array, group_bounds as
 * the host array of ocnn_pair_plan_lists).  Weights stay in registers, a workgroup serves 32
 * output channels over many tiles, results are added in a fixed order.  f16 / bf16, cin in
 * {32, 64, 96, 128}, cout % 32 == 0, K <= 27; same result as ocnn_conv_gather. */
int ocnn_conv_gather_sparse_supported(int dtype, int64_t rows_in, int K, int cin, int cout,
                                      int plan_max_distinct);
int64_t ocnn_conv_gather_sparse_workspace_bytes(int cin, int cout);
int ocnn_conv_gather_sparse(int dtype, const void* in, int64_t rows_in, const int32_t* uptr,
                            const int32_t* urows, int plan_max_distinct, int64_t plan_total,
                            const int32_t* cptr, const uint32_t* ent, int64_t n_blocks,
                            int max_blocks, const int32_t* lists, int n_lists,
                            const int32_t* group_bounds, int64_t rows_out, int K, const void* w,
                            int cin, int cout, int w_transposed, int reverse_slots, const void* bias,
                            void* out, void* workspace, int64_t workspace_bytes, void* stream);

/* Weight gradient over the pair plan of a sparse table (the counterpart of
 * ocnn_conv_gather_sparse; same sums as ocnn_conv_wgrad):
 *   D[k][i][j] = sum over the table rows r with table[r][k] >= 0 of a[table[r][k]][i] * b[r][j]
 * a: (rows_a, ca), the rows the table points at; b: (rows_b, cb), the rows of the table,
 * cb <= 96; ca, cb multiples of 32; f16 / bf16.  out: (K, ca, cb) with a_major, (K, cb, ca)
 * without.  lists and list_count are the HOST arrays of ocnn_pair_plan_lists.  A workgroup
 * keeps the fp32 sums of all lists for 32 a-channels in registers over a range of tiles; the
 * ranges are added in a fixed order. */
int ocnn_conv_wgrad_sparse_supported(int dtype, int64_t rows_a, int64_t rows_b, int K, int ca, int cb,
                                     int plan_max_distinct);
int64_t ocnn_conv_wgrad_sparse_workspace_bytes(int64_t rows_b, int ca, int cb);
int ocnn_conv_wgrad_sparse(int dtype, const void* a, int64_t rows_a, int ca, const void* b,
                           int64_t rows_b, int cb, const int32_t* uptr, const int32_t* urows,
                           int plan_max_distinct, int64_t plan_total, const int32_t* cptr,
                           const uint32_t* ent, int64_t n_blocks, const int32_t* lists,
                           const int64_t* list_count, int n_lists, int K, int a_major, void* out,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* out (rows, cout) = in (rows, cin) W (+ bias): ocnn_conv_gather with the one-slot identity
 * table, the form that the 2x2x2 stride-2 layers over all nodes take on the (parents, 8 C)
 * view of the children (ocnn/nn/octree_conv.py:115-168 with neigh[p] = 8p .. 8p+7).
 * w: (cin, cout), or (cout, cin) with w_transposed.  f16 / bf16, cin % 64 == 0 (<= 1024),
 * cout % 128 == 0; workspace cin * cout * 2 bytes. */
int ocnn_conv_dense_supported(int dtype, int64_t rows, int cin, int cout);
int ocnn_conv_dense(int dtype, const void* in, int64_t rows, const void* w, int cin, int cout,
                    int w_transposed, const void* bias, void* out, void* workspace,
                    int64_t workspace_bytes, void* stream);

/* The same GEMM, and its weight gradient gw (ca, cb) [or (cb, ca)] = x^T g, with what is
 * reused kept in registers by persistent workgroups (weights, resp. the fp32 sums), so that
 * each tensor crosses L2 once: cin in {64, 128, 256, 512}, cout % 128 == 0; weight gradient
 * for any ca, cb that are multiples of 8 (summed in blocks of 512 x 128, 256 x 256 or
 * 128 x 512 channel pairs, whichever covers ca x cb with the fewest; the channels a block
 * has past ca or cb are staged as zeros and not written). */
int ocnn_conv_dense_rw_supported(int dtype, int64_t rows, int cin, int cout);
int ocnn_conv_dense_rw(int dtype, const void* in, int64_t rows, const void* w, int cin, int cout,
                       int w_transposed, const void* bias, void* out, void* workspace,
                       int64_t workspace_bytes, void* stream);
int ocnn_conv_dense_wgrad_rw_supported(int dtype, int64_t rows, int ca, int cb);
int64_t ocnn_conv_dense_wgrad_rw_workspace_bytes(int ca, int cb);
int ocnn_conv_dense_wgrad_rw(int dtype, const void* x, const void* g, int64_t rows, int ca, int cb,
                             int out_transposed, void* gw, void* workspace,
                             int64_t workspace_bytes, void* stream);

/* The two of them with the rows of an operand taken through an index: row i of the GEMM's
 * input (of x, of g) is row index[i] of a tensor with rows_in (rows_x, rows_g) rows; a NULL
 * index means the operand's own rows 0 .. rows - 1, as above.  This is how the stride-2 layers
 * over all nodes read the rows of the non-empty nodes out of a tensor padded to all nodes
 * without a depad pass (the reference depads first: ocnn/nn/octree_conv.py:419-420, 450-451,
 * ocnn/nn/octree_pad.py:32-39).  The GEMM's result likewise: with out_index, row i is written to
 * row out_index[i] of `out`, a tensor of rows_out rows (NULL: out has the `rows` rows of the
 * result); the rows no entry names are not touched, ocnn_pad with data = NULL zeroes them: the
 * reference's octree_pad after the product (ocnn/nn/octree_conv.py:388-389,
 * ocnn/nn/octree_pad.py:13-29) without the copy. */
int ocnn_conv_dense_rw_indexed(int dtype, const void* in, int64_t rows_in, const int32_t* row_index,
                               int64_t rows, const void* w, int cin, int cout, int w_transposed,
                               const void* bias, void* out, int64_t rows_out,
                               const int32_t* out_index, void* workspace, int64_t workspace_bytes,
                               void* stream);
int ocnn_conv_dense_wgrad_rw_indexed(int dtype, const void* x, int64_t rows_x, const int32_t* x_index,
                                     const void* g, int64_t rows_g, const int32_t* g_index,
                                     int64_t rows, int ca, int cb, int out_transposed, void* gw,
                                     void* workspace, int64_t workspace_bytes, void* stream);

/* Weight gradient, ocnn/nn/octree_conv.py:170-202 (weight_gemm) and
 * ocnn/nn/kernels/conv_bwd_implicit_gemm_splitk.py:94-184,294-306:
 * gw[k][a][b] = sum_i [t[i][k] >= 0] x[t[i][k]][a] * g[i][b], computed as
 * split-K partial sums over row ranges (fp32) followed by a fixed-order
 * reduction - no atomics, bit-reproducible.  x: (rows_x, ca); g: (rows, cb);
 * gw: (K, ca, cb) in `dtype`, or (K, cb, ca) when out_transposed != 0 (the
 * deconvolution's weight layout, ocnn/nn/octree_conv.py:287-290). */
int64_t ocnn_conv_wgrad_workspace_bytes(int64_t rows, int K, int ca, int cb);
/* The same with the room an fp32 layer needs to run on the MFMA kernels as three bf16
 * pieces (hi/lo split of both operands, about 1e-5 relative; without that room fp32 runs on
 * the plain kernel). */
int64_t ocnn_conv_wgrad_workspace_bytes_for(int dtype, int64_t rows_x, int64_t rows, int K,
                                            int ca, int cb);
int ocnn_conv_wgrad(int dtype, const void* x, int64_t rows_x, const void* g,
                    const int32_t* table, int64_t rows, int K, int ca, int cb,
                    int out_transposed, void* gw, void* workspace,
                    int64_t workspace_bytes, void* stream);

/* ocnn_conv_wgrad over a tile plan of the same table, for ca = cb = 32 and for ca, cb
 * multiples of 64 up to 1024, summed in 64 x 64 blocks of channel pairs (same
 * reference lines, same result up to the fp32 summation order, which is fixed).
 * Per tile the distinct x rows and the g rows are staged once in LDS; persistent
 * workgroups keep the sums of all K slots in accumulator registers over a range
 * of tiles.  plan_max_distinct must be <= 415; ..._supported() tells.
 * fp32 tensors run as two bf16 pieces each (x = hi + lo): three passes of the bf16
 * kernel (hi hi, hi lo, lo hi) into three sets of sums and one reduction, about 1e-5
 * relative; the workspace then also holds the pieces: ..._workspace_bytes_for(). */
int ocnn_conv_wgrad_planned_supported(int dtype, int64_t rows_x, int64_t rows, int K, int ca,
                                      int cb, int plan_max_distinct);
int64_t ocnn_conv_wgrad_planned_workspace_bytes(int K, int ca, int cb);   /* f16 / bf16 */
int64_t ocnn_conv_wgrad_planned_workspace_bytes_for(int dtype, int64_t rows_x, int64_t rows, int K,
                                                    int ca, int cb);
int ocnn_conv_wgrad_planned(int dtype, const void* x, int64_t rows_x, const void* g,
                            const uint16_t* loc, const int32_t* uptr, const int32_t* urows,
                            int plan_max_distinct, int64_t plan_total, int64_t rows, int K,
                            int ca, int cb, int out_transposed, void* gw, void* workspace,
                            int64_t workspace_bytes, void* stream);

/* Depth-wise engine, ocnn/nn/octree_dwconv.py:30-118.  w: (K, c).
 * fwd : out[i][c] = sum_k in[t[i][k]][c] * w[k'][c]   (k' = K-1-k if
 *       reverse_slots; with a transposed or mirrored table this is also the
 *       data gradient);
 * wgrad: gw[k][c] = sum_i x[t[i][k]][c] * g[i][c] (two-pass, deterministic). */
int ocnn_dwconv_gather(int dtype, const void* in, int64_t rows_in,
                       const int32_t* table, int64_t rows_out, int K,
                       const void* w, int channels, int reverse_slots,
                       const void* bias, void* out, void* stream);
int64_t ocnn_dwconv_wgrad_workspace_bytes(int64_t rows, int K, int channels);
int ocnn_dwconv_wgrad(int dtype, const void* x, int64_t rows_x, const void* g,
                      const int32_t* table, int64_t rows, int K, int channels,
                      void* gw, void* workspace, int64_t workspace_bytes,
                      void* stream);

/* The depth-wise engine over the tile plan of the table (same reference lines, same
 * results up to the fp32 summation order, which is fixed): the distinct rows of a tile
 * are staged once in LDS, 64 channels at a time, and the products run on the 4x4x4 matrix
 * instruction.  f16 / bf16, channels a multiple of 64, plan_max_distinct <= 416, K in
 * {27, 9, 8, 3}.  A non-finite input value reaches the other three channels of its group
 * of four (0 x inf inside the instruction). */
int ocnn_dwconv_gather_planned_supported(int dtype, int64_t rows_in, int K, int channels,
                                         int plan_max_distinct);
int ocnn_dwconv_gather_planned(int dtype, const void* in, int64_t rows_in, const uint16_t* loc,
                               const int32_t* uptr, const int32_t* urows, int plan_max_distinct,
                               int64_t plan_total, int64_t rows_out, int K, const void* w,
                               int channels, int reverse_slots, const void* bias, void* out,
                               void* stream);
int ocnn_dwconv_wgrad_planned_supported(int dtype, int64_t rows_x, int64_t rows, int K,
                                        int channels, int plan_max_distinct);
int64_t ocnn_dwconv_wgrad_planned_workspace_bytes(int K, int channels);
int ocnn_dwconv_wgrad_planned(int dtype, const void* x, int64_t rows_x, const void* g,
                              const uint16_t* loc, const int32_t* uptr, const int32_t* urows,
                              int plan_max_distinct, int64_t plan_total, int64_t rows, int K,
                              int channels, void* gw, void* workspace, int64_t workspace_bytes,
                              void* stream);

/* Batch normalisation over the rows of a (rows, c) matrix with the ReLU of the
 * conv-bn-relu blocks fused in (ocnn/modules/modules.py:32-99: OctreeConvBn, OctreeConvBnRelu,
 * OctreeDeconvBnRelu use torch.nn.BatchNorm1d + ReLU): per-channel mean, biased variance and
 * 1 / sqrt(var + eps) of x; y = (x - mean) * invstd * gamma + beta [then max(., 0)]; and the
 * gradient dx, dgamma, dbeta (training = 1: statistics of this batch; 0: fixed statistics;
 * dx may be NULL).  gamma / beta (dtype param_dtype) may be NULL (no affine part); the
 * statistics kernel also moves running_mean / running_var (dtype running_dtype, may be NULL)
 * towards the batch statistics by `factor`, the running variance towards the unbiased one
 * (torch.nn.functional.batch_norm) and adds one to *batches_tracked (device, may be NULL: the
 * module's num_batches_tracked); dgamma / dbeta are fp32, grad_gamma / grad_beta the same
 * sums in param_dtype (may be NULL).  fp32 arithmetic, two-level reductions with a fixed order.
 * channels a multiple of 16 bytes of elements.  residual (may be NULL): a tensor like x added
 * to the normalised values before the ReLU, each summand rounded to the dtype first (the
 * tail of a residual block, ocnn/modules/resblocks.py:96-99); the backward pass then takes the
 * forward output y for the ReLU's mask and writes the residual's gradient to d_residual
 * (both may be NULL). */
int ocnn_batch_norm_supported(int dtype, int64_t rows, int channels);
int64_t ocnn_batch_norm_workspace_bytes(int channels);
int ocnn_batch_norm_stats(int dtype, const void* x, int64_t rows, int channels, float eps,
                          float* mean, float* var, float* invstd, void* running_mean,
                          void* running_var, int running_dtype, float factor,
                          int64_t* batches_tracked, void* workspace, int64_t workspace_bytes,
                          void* stream);
int ocnn_batch_norm_apply(int dtype, const void* x, int64_t rows, int channels, const float* mean,
                          const float* invstd, const void* gamma, const void* beta,
                          int param_dtype, int relu, const void* residual, void* y, void* stream);
int ocnn_batch_norm_backward(int dtype, const void* x, const void* dy, int64_t rows, int channels,
                             const float* mean, const float* invstd, const void* gamma,
                             const void* beta, int param_dtype, int relu, int training,
                             const void* y, void* dx, void* d_residual, float* dgamma, float* dbeta,
                             void* grad_gamma, void* grad_beta, void* workspace,
                             int64_t workspace_bytes, void* stream);

/* Key search, ocnn/octree/octree.py:448-488 (search_key / search_xyzb): out[i] = position of
 * query[i] in the ascending `keys`, or -1.  ocnn_search_points takes float (x, y, z, b) rows,
 * truncates and encodes them like xyz2key (ocnn/octree/shuffled_key.py:60-90) and, with
 * bound_check, rejects coordinates outside [0, 2^depth) (ocnn/nn/octree_interp.py:38-42). */
int ocnn_search_key(const int64_t* keys, int64_t n, const int64_t* query, int64_t m,
                    int64_t* out, void* stream);
int ocnn_search_points(const float* pts, int64_t m, int depth, const int64_t* keys, int64_t n,
                       int bound_check, int32_t* out, void* stream);

/* Trilinear interpolation, ocnn/nn/octree_interp.py:49-103 (octree_linear_pts), in two steps:
 * the 8 neighbour rows idx (m, 8) (-1 = none), their weights w (m, 8) and the weight sum
 * norm (m) of every point (lines 60-88), then out = (sum_j w_j data[idx_j]) / (norm + 1e-12)
 * as ocnn_csr_rows with 8 entries per row (lines 90-102).  ocnn_csr_rows is the product of
 * a sparse matrix in row form with a dense one, out[r] = (sum_e val[e] data[col[e]]) /
 * (rowdiv[r] + 1e-12): entries rowptr[r] .. rowptr[r+1]-1, or kfixed per row when rowptr is
 * NULL; val NULL = ones, rowdiv NULL = no division, col < 0 = no entry.  With the transposed
 * matrix it is the gradient with respect to data (no atomics, fixed summation order). */
int ocnn_interp_linear_prepare(const float* pts, int64_t m, int depth, const int64_t* keys,
                               int64_t n, int bound_check, int32_t* idx, float* w, float* norm,
                               void* stream);
/* ocnn_search_points and ocnn_interp_linear_prepare for the nodes of an octree layer, found by
 * walking down the tree instead of searching the layer's keys (same results: the node's row,
 * among all nodes of `depth` or, with nempty, among the non-empty ones, or -1): the children of
 * the c-th non-empty node of a layer are the nodes 8 c .. 8 c + 7 of the next.  h_children: host
 * array of depth + 1 device pointers, the octree's children arrays (layers min(depth,
 * full_depth) .. depth are read; the last only with nempty). */
int ocnn_locate_points(const float* pts, int64_t m, const int32_t* const* h_children, int depth,
                       int full_depth, int batch_size, int nempty, int bound_check, int32_t* out,
                       void* stream);
int ocnn_interp_linear_locate(const float* pts, int64_t m, const int32_t* const* h_children,
                              int depth, int full_depth, int batch_size, int nempty,
                              int bound_check, int32_t* idx, float* w, float* norm, void* stream);
int ocnn_csr_rows(int dtype, const int32_t* rowptr, int kfixed, const int32_t* col,
                  const float* val, const void* data, int channels, const float* rowdiv,
                  void* out, int64_t rows, void* stream);

/* The transposed matrix in that row form (what torch.sparse.mm's backward needs,
 * ocnn/nn/octree_interp.py:98-102, here without atomics): entry (p, j) of idx (points, k) with
 * idx >= 0 becomes an entry of data row idx[p, j] with column p and value w[p, j] /
 * (norm[p] + 1e-12) (norm NULL: no division; w NULL: ones; both NULL: val NULL, nothing stored).  The entries
 * of a row keep the order of the points.  rowptr: rows + 1 values; col, val: capacity points * k,
 * the first rowptr[rows] of them used. */
int64_t ocnn_csr_transpose_workspace_bytes(int64_t entries);
int ocnn_csr_transpose(const int32_t* idx, const float* w, const float* norm, int64_t points,
                       int k, int64_t rows, void* workspace, int64_t workspace_bytes,
                       int32_t* rowptr, int32_t* col, float* val, void* stream);

/* 2x2x2 max pooling, ocnn/nn/octree_pool.py:16-65.
 * ocnn_max_pool: maximum over the children 8p .. 8p+7 of the p-th non-empty node (first on
 * ties) and its index (indices (parents, c) int64).  fine_child = children of the fine
 * level when data holds non-empty nodes only (an empty child counts as -inf), NULL when it
 * holds all nodes; coarse_child = children of the coarse level when the output has a row
 * for every coarse node (zeros for empty ones, the octree_pad of line 36), NULL when it
 * has one per non-empty node.
 * ocnn_max_unpool: out row r = child q % 8 of parent q / 8 (q = out_node[r] or r) takes
 * src[src_row[p] or p] where indices say so, else 0 (lines 40-65; also d pool / d data).
 * ocnn_max_gather: out[p] = src[row of child 8p + indices[p]] (d unpool / d data). */
int ocnn_max_pool(int dtype, const void* data, const int32_t* fine_child,
                  const int32_t* coarse_child, int64_t out_rows, int channels, void* out,
                  int64_t* indices, void* stream);
int ocnn_max_unpool(int dtype, const void* src, const int64_t* indices, const int32_t* out_node,
                    const int32_t* src_row, int64_t out_rows, int channels, void* out,
                    void* stream);
int ocnn_max_gather(int dtype, const void* src, const int64_t* indices,
                    const int32_t* fine_child, int64_t parents, int channels, void* out,
                    void* stream);

/* ocnn/nn/octree_pad.py:13-39.  pad: out (n, c) = val except out[q] =
 * data[children[q]] where children[q] >= 0 (data NULL: only the rows with
 * children[q] < 0 are written, for a result whose other rows are in place
 * already); depad: out[children[q]] = data[q]. */
int ocnn_pad(int dtype, const void* data, const int32_t* children, int64_t n,
             int channels, float val, void* out, void* stream);
int ocnn_depad(int dtype, const void* data, const int32_t* children, int64_t n,
               int channels, void* out, void* stream);

/* Column sum (grad_bias = grad.sum(0), ocnn/nn/kernels/
 * conv_bwd_implicit_gemm_splitk.py:343-345), two-pass deterministic.
 * workspace: ocnn_colsum_workspace_bytes(rows, channels). */
int64_t ocnn_colsum_workspace_bytes(int64_t rows, int channels);
int ocnn_colsum(int dtype, const void* g, int64_t rows, int channels, void* out,
                void* workspace, int64_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* OCNN_HIP_H_ */
