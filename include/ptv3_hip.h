/* C ABI of libptv3_hip.so — hand-written gfx950 kernels for the Point Transformer V3
 * forward path.
 *
 * Conventions
 *   - every pointer named *_dev / without suffix is DEVICE memory unless the comment says
 *     "host"; sizes are element counts unless they end in _bytes
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued asynchronously on it
 *   - no entry point allocates or frees device memory or synchronises the device:
 *     outputs and workspaces are the caller's (query the size with *_workspace_bytes)
 *   - return value: 0 ok; < 0 argument error (PTV3_E*); > 0 a hipError_t from a launch
 *   - dtype codes: 0 = float32, 1 = float16, 2 = bfloat16
 *
 * The reference has no native interface; each entry point names the Python lines whose
 * device work it replaces (paths relative to the reference checkout).
 */
#ifndef PTV3_HIP_H
#define PTV3_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTV3_OK 0
#define PTV3_EINVAL (-1)    /* null pointer, negative size, unknown enum */
#define PTV3_EDEPTH (-2)    /* depth outside 1..16 or code wider than 63 bits (model.py:103,108) */
#define PTV3_EWORKSPACE (-3) /* workspace smaller than *_workspace_bytes says */
#define PTV3_ESHAPE (-4)    /* channel / head / patch shape the kernels do not cover */
#define PTV3_ESTATIC (-5)   /* input larger than the fixed on-device buffer of a *_static entry point */

#define PTV3_F32 0
#define PTV3_F16 1
#define PTV3_BF16 2

#define PTV3_ORDER_Z 0
#define PTV3_ORDER_Z_TRANS 1
#define PTV3_ORDER_HILBERT 2
#define PTV3_ORDER_HILBERT_TRANS 3

int ptv3_version(void);
const char *ptv3_strerror(int rc);

/* serialization/default.py:8-24 -> z_order.py:66-101, hilbert.py:91-198.
 * grid_coord (n,3) int32; batch (n,) int64 or NULL; order_ids: HOST array of k PTV3_ORDER_*;
 * code (k,n) int64, row r holds order_ids[r]. All k orders are produced in one pass. */
int ptv3_encode(const int32_t *grid_coord, const int64_t *batch, int64_t n, int depth,
                const int32_t *order_ids_host, int k, int64_t *code, void *stream);

/* serialization/default.py:27-39 -> z_order.py:104-126, hilbert.py:201-303 (the inverse of ptv3_encode for one
 * order). code (n,) int64; grid_coord (n,3) int64 out (the reference returns int64 coordinates);
 * batch (n,) int64 out or NULL: code >> 3*depth. */
int ptv3_decode(const int64_t *code, int64_t n, int depth, int order_id, int64_t *grid_coord,
                int64_t *batch, void *stream);

/* model.py:100 (depth = bit length of the largest coordinate) and :162-164 (sparse_shape):
 * per-axis maximum of grid_coord (n,3) int32 into out3 (3 int32, device). n >= 1. */
int ptv3_grid_max(const int32_t *grid_coord, int64_t n, int32_t *out3, void *stream);

/* Voxelisation in front of the model (what Pointcept's data pipeline does on the host before
 * PointTransformerV3.forward, model.py:966-973, sees a batch; model.py:88-96 is the model's own
 * fallback for grid_coord alone): per scene, grid_coord = floor((coord - scene minimum) / grid_size),
 * and the first point in input order of every voxel is kept. coord (n,3) float32, offset (n_scenes,)
 * int64 cumulative scene ends, all on the device. Outputs, sized for n by the caller: grid_coord
 * (m,3) int32 and index (m,) int64 of the kept points in input order, inverse (n,) int64 = position
 * of every input point's voxel among the kept ones (or NULL), offset_out (n_scenes,) int64 = scene
 * ends of the kept points, counts (2,) int64 on the device = {m, status}; status 1 means a grid
 * coordinate needs more than 16 bits (the serialization's limit, model.py:108) and the rest is
 * meaningless. n < 2^30. pick_seed 0 keeps the first point in input order (GridSample's test mode); any other
 * value keeps a member of every voxel drawn uniformly, a different draw per seed (its train mode; the
 * random stream is this library's own, not numpy's). */
size_t ptv3_voxelize_workspace_bytes(int64_t n, int n_scenes);
int ptv3_voxelize(const float *coord, int64_t n, const int64_t *offset, int n_scenes, float grid_size,
                  int32_t *grid_coord, int64_t *index, int64_t *inverse, int64_t *offset_out,
                  int64_t *counts, uint32_t pick_seed, void *workspace, size_t workspace_bytes, void *stream);

/* model.py:35-40 (offset2batch): scene id of each of the n points from the cumulative scene ends
 * offset (n_scenes,) int64 on the device, n = offset[n_scenes - 1] known to the caller. */
int ptv3_offset2batch(const int64_t *offset, int n_scenes, int64_t n, int64_t *batch, void *stream);

/* model.py:119-126 and :667-674: per-row ascending argsort of (k,n) int64 codes plus the
 * inverse permutation. Only the low `key_bits` bits are sorted on (the rest must be equal
 * across a row, e.g. zero); ties keep their input order. */
size_t ptv3_argsort_workspace_bytes(int64_t n, int k);
int ptv3_argsort(const int64_t *code, int64_t n, int k, int key_bits, int64_t *order,
                 int64_t *inverse, void *workspace, size_t workspace_bytes, void *stream);

/* model.py:392-437. ptv3_pad_sizes is host-only arithmetic on a HOST copy of `offset`
 * (nb cumulative scene ends): total padded length and number of sequences.
 * ptv3_pad_index fills pad (n_pad,), unpad (n,), cu_seqlens (n_seq+1,) int32 from the
 * DEVICE offset; workspace >= ptv3_pad_index_workspace_bytes(nb). */
int ptv3_pad_sizes(const int64_t *offset_host, int nb, int64_t patch, int64_t *n_pad,
                   int64_t *n_seq);
size_t ptv3_pad_index_workspace_bytes(int nb);
int ptv3_pad_index(const int64_t *offset, int nb, int64_t patch, int64_t n, int64_t n_pad,
                   int64_t n_seq, int64_t *pad, int64_t *unpad, int32_t *cu_seqlens,
                   void *workspace, size_t workspace_bytes, void *stream);

/* model.py:452-453,456,484 folded into two int32 tables for one serialization order:
 * slot_src[i] = order[pad[i]] (row to read for padded slot i) and
 * slot_dst[i] = that row again when i is the row's own slot (unpad[inverse[row]] == i),
 * else -1 (filler slots only lend keys/values, model.py:412-423). */
int ptv3_attn_slots(const int64_t *order_row, const int64_t *inverse_row, const int64_t *pad,
                    const int64_t *unpad, int64_t n_pad, int32_t *slot_src, int32_t *slot_dst,
                    void *stream);

/* model.py:456-484 (flash_attn_varlen_qkvpacked_func call at :476-482 and the torch
 * fallback :460-474): non-causal softmax(q k^T * scale) v inside each sequence, per head.
 * qkv (n_rows, 3*C) with channel layout [3][H][D], D = C/H; rows are fetched through
 * slot_src and results written to out[slot_dst[i]] (n_rows, C) when slot_dst[i] >= 0.
 * cu_seqlens (n_seq+1,) int32 in padded-slot units; no sequence is longer than max_seqlen.
 * D = 16 in fp16 / bf16 with sequences of up to 2368 keys (every released PTv3 configuration) runs on the MFMA
 * kernel; fp32, D = 8, 32 or 64, and longer sequences run on a thread-per-query kernel in fp32 arithmetic
 * (an order of magnitude slower). Other head dims: PTV3_ESHAPE. */
int ptv3_patch_attn_fwd(const void *qkv, int dtype, int64_t n_rows, int channels, int heads,
                        const int32_t *slot_src, const int32_t *slot_dst,
                        const int32_t *cu_seqlens, int64_t n_seq, int64_t max_seqlen,
                        float scale, void *out, void *stream);

/* The same with the relative position bias of model.py:297-316, :468-469 (fp32 only: the reference
 * applies it on its non-fused path, in float): score(query i, key j, head h) +=
 * sum over the axes a of rpe_table[a * R + clamp(g_i[a] - g_j[a], -pos_bnd, pos_bnd) + pos_bnd][h],
 * R = 2 * pos_bnd + 1; grid_coord (n_rows, 3) int32 in point order, rpe_table (3 * R, heads) fp32,
 * pos_bnd <= 128; D = C / heads = 8, 16, 32 or 64. dropout_p, dropout_seed: attention dropout as in
 * ptv3_patch_attn_fwd_lse (0, 0 for none). */
int ptv3_patch_attn_rpe_fwd(const float *qkv, int64_t n_rows, int channels, int heads,
                            const int32_t *slot_src, const int32_t *slot_dst,
                            const int32_t *cu_seqlens, int64_t n_seq, int64_t max_seqlen, float scale,
                            const int32_t *grid_coord, const float *rpe_table, int pos_bnd, float dropout_p,
                            uint32_t dropout_seed, float *out, void *stream);

/* ptv3_patch_attn_fwd for training (D = 16 only, like the backward entry points). fp16 / bf16: also keeps what the backward pass needs, lse (heads, n_pad)
 * fp32, lse[h][slot] = log2 of the sum over the slot's sequence of 2^(score * log2(e)) for every real slot
 * (filler slots are left unwritten); fp32: lse may be NULL (the backward recomputes it). n_pad =
 * cu_seqlens[n_seq]. dropout_p in [0, 1): attention dropout (model.py:470, :480) -- probability (head, query
 * slot, key slot) is zeroed when a hash of (dropout_seed, head, query slot, key slot) falls below
 * dropout_p * 2^32, the others are divided by 1 - dropout_p; the backward entry points take the same two
 * values and recompute the same bits. */
int ptv3_patch_attn_fwd_lse(const void *qkv, int dtype, int64_t n_rows, int channels, int heads,
                            const int32_t *slot_src, const int32_t *slot_dst, const int32_t *cu_seqlens,
                            int64_t n_seq, int64_t max_seqlen, int64_t n_pad, float scale, float dropout_p,
                            uint32_t dropout_seed, void *out, float *lse, void *stream);

/* Backward of ptv3_patch_attn_fwd: what autograd derives for model.py:456-484 (the backward of the
 * flash_attn_varlen_qkvpacked_func call at :476-482 and of the row gathers around it). out is the
 * forward result, dout its gradient (n_rows, C); dqkv (n_rows, 3*C) receives [dq | dk | dv] per row,
 * every element written. Filler slots take no gradient as queries; as keys their share is added to
 * the row they repeat. n_pad = cu_seqlens[n_seq], the number of slots. lse: what ptv3_patch_attn_fwd_lse
 * wrote for the same inputs (fp16 / bf16 only), or NULL to have it recomputed. dropout_p, dropout_seed: as
 * given to the forward call. */
size_t ptv3_patch_attn_bwd_workspace_bytes(int dtype, int64_t n_pad, int channels, int heads);
int ptv3_patch_attn_bwd(const void *qkv, const void *out, const void *dout, int dtype, int64_t n_rows,
                        int channels, int heads, const int32_t *slot_src, const int32_t *slot_dst,
                        const int32_t *cu_seqlens, int64_t n_seq, int64_t max_seqlen, int64_t n_pad,
                        float scale, const float *lse, float dropout_p, uint32_t dropout_seed, void *dqkv,
                        void *workspace, size_t workspace_bytes, void *stream);

/* Backward of ptv3_patch_attn_rpe_fwd (fp32): as ptv3_patch_attn_bwd, with the relative position bias of
 * model.py:297-316 in the scores; drpe_table (3 * R, heads) fp32 is accumulated into (zero it first):
 * entry [a * R + c][h] += sum of dS(h, i, j) over the pairs (i, j) whose clamped offset along axis a is c.
 * grid_coord == NULL: exactly ptv3_patch_attn_bwd. */
int ptv3_patch_attn_rpe_bwd(const void *qkv, const void *out, const void *dout, int dtype, int64_t n_rows,
                            int channels, int heads, const int32_t *slot_src, const int32_t *slot_dst,
                            const int32_t *cu_seqlens, int64_t n_seq, int64_t max_seqlen, int64_t n_pad,
                            float scale, const float *lse, float dropout_p, uint32_t dropout_seed,
                            const int32_t *grid_coord, const float *rpe_table, int pos_bnd, float *drpe_table,
                            void *dqkv, void *workspace, size_t workspace_bytes, void *stream);

/* spconv.SubMConv3d's index generation (call sites model.py:546-552, :767-774, tensor built
 * at :165-172). indices (n,4) int32 [batch,x,y,z], coordinates in [0, 65535];
 * nbr int32, entry (voxel i, tap t = (kx*ks+ky)*ks+kz) = row of the voxel at
 * (b, x+kx-ks/2, y+ky-ks/2, z+kz-ks/2) or -1; stored voxel-major (n, ks^3) when tap_major == 0,
 * tap-major (ks^3, n) otherwise (the layout the convolution kernels read coalesced; every
 * function below that takes nbr also takes this flag). ks is 3 or 5. */
size_t ptv3_kmap_workspace_bytes(int64_t n);
int ptv3_kmap_build(const int32_t *indices, int64_t n, int ks, int tap_major, int32_t *nbr,
                    void *workspace, size_t workspace_bytes, void *stream);

/* spconv.SubMConv3d forward (same call sites): out[i] = bias + sum_k W[:,k,:] feat[nbr[i][k]].
 * feat (n,cin), weight (cout, V, cin) (spconv 2.x KRSC layout flattened over the taps),
 * bias (cout,) or NULL, out (n,cout); all of `dtype`, accumulation in fp32. */
int ptv3_subm_conv_fwd(const void *feat, int dtype, int64_t n, int cin, const int32_t *nbr,
                       int taps, int tap_major, const void *weight, const void *bias, int cout,
                       void *out, void *stream);

/* Weight gradient of spconv.SubMConv3d (same call sites): dweight[co][t][ci] = sum over voxels i with
 * nbr[t][i] >= 0 of dout[i][co] * feat[nbr[t][i]][ci]. nbr is tap-major (taps, n); dweight
 * (cout, taps, cin) fp32, every element written; dbias (cout,) fp32 or NULL: sum over the voxels of dout
 * (fp16 / bf16 with cin and cout multiples of 8 only, PTV3_ESHAPE otherwise). The input gradient needs
 * no kernel of its own: it is ptv3_subm_conv_fwd of dout with weight'[ci][t][co] = weight[co][taps-1-t][ci]. */
size_t ptv3_subm_conv_wgrad_workspace_bytes(int dtype, int64_t n, int cin, int cout, int taps);
int ptv3_subm_conv_wgrad(const void *feat, const void *dout, int dtype, int64_t n, int cin, int cout,
                         const int32_t *nbr, int taps, float *dweight, float *dbias, void *workspace,
                         size_t workspace_bytes, void *stream);

/* The same weight gradient from the tap-major pair lists the forward pair kernels use (ptv3_conv_plan_*)
 * instead of the neighbour map: work-groups take ranges of a tap's own pairs, so nothing is compacted and the
 * ranges are equally long whatever the tap's density. pair_out[q] is the output voxel of pair q
 * (ptv3_conv_plan_pair_out makes it from the plan's row_ptr and pair_slot); fp16 / bf16 with cin and cout
 * multiples of 8 only; workspace as ptv3_subm_conv_wgrad_workspace_bytes says. The centre tap must pair every
 * voxel with itself (true for a submanifold convolution): dbias is summed over its pairs. */
int ptv3_conv_plan_pair_out(const int32_t *row_ptr, const int32_t *pair_slot, int64_t n, int64_t n_pairs,
                            int32_t *pair_out, void *stream);
int ptv3_subm_conv_wgrad_pairs(const void *feat, const void *dout, int dtype, int64_t n, int cin, int cout,
                               const int32_t *tap_ptr, const int32_t *pair_in, const int32_t *pair_out, int taps,
                               float *dweight, float *dbias, void *workspace, size_t workspace_bytes, void *stream);

/* Sparse-pair form of the same convolution, for maps where most taps of most voxels are empty
 * (surface scans: 2-13 of 27 taps active). ptv3_conv_plan_count derives from nbr (n,taps) the
 * number of active (input, output) pairs per tap (tap_ptr, taps+1 int32, exclusive) and in total
 * (n_pairs, device int64); after reading n_pairs on the host, ptv3_conv_plan_fill writes
 * row_ptr (n+1 int32: first output slot of every voxel), and per tap-major pair its input row
 * (pair_in) and output slot (pair_slot), both (n_pairs,) int32. Same workspace for both calls,
 * >= ptv3_conv_plan_workspace_bytes(n, taps); taps <= 128.
 * ptv3_subm_conv_pairs_fwd multiplies every pair's input row by its tap's weight matrix with
 * fully populated MFMA tiles into y (n_pairs, cout) and sums each voxel's slots (+bias) into
 * out (n, cout). fp16/bf16 only; cin % 16 == 0, cout % 8 == 0. */
size_t ptv3_conv_plan_workspace_bytes(int64_t n, int taps);
int ptv3_conv_plan_count(const int32_t *nbr, int64_t n, int taps, int tap_major, int32_t *tap_ptr,
                         int64_t *n_pairs, void *workspace, size_t workspace_bytes, void *stream);
int ptv3_conv_plan_fill(const int32_t *nbr, int64_t n, int taps, int tap_major, const int32_t *tap_ptr,
                        int32_t *row_ptr, int32_t *pair_in, int32_t *pair_slot, void *workspace,
                        size_t workspace_bytes, void *stream);
/* The same pair lists straight from the voxel coordinates (indices as for ptv3_kmap_build), without
 * a stored neighbour map: bit-identical to ptv3_conv_plan_count / _fill applied to the map
 * ptv3_kmap_build returns. The count call builds the voxel hash in the workspace, the fill call
 * (after n_pairs has been read on the host) reuses it: same workspace, untouched in between,
 * >= ptv3_kmap_plan_workspace_bytes(n, ks); ks is 3 or 5. Replaces spconv's indice-pair generation
 * for SubMConv3d (call sites model.py:546-552, :767-774). */
size_t ptv3_kmap_plan_workspace_bytes(int64_t n, int ks);
int ptv3_kmap_plan_count(const int32_t *indices, int64_t n, int ks, int32_t *tap_ptr, int64_t *n_pairs,
                         void *workspace, size_t workspace_bytes, void *stream);
int ptv3_kmap_plan_fill(const int32_t *indices, int64_t n, int ks, const int32_t *tap_ptr,
                        int32_t *row_ptr, int32_t *pair_in, int32_t *pair_slot, void *workspace,
                        size_t workspace_bytes, void *stream);
/* The 3x3x3 pair lists of a voxel set from its 5x5x5 lists (a 5x5x5 stem and 3x3x3 blocks on the same
 * level, model.py:767-774 and :546-552): the inner 27 taps of the 5x5x5 neighbourhood are the 3x3x3
 * neighbourhood, so one voxel hash and one neighbour search serve both. Bit-identical to
 * ptv3_kmap_plan_count / _fill with ks = 3.
 * _inner_count reads what ptv3_kmap_plan_count(ks = 5) left in its workspace (workspace5, untouched
 * since) and writes found3 (n,) int32 [bit t: voxel has tap t], row_cnt3 (n,) int32 [pairs per voxel],
 * tap_ptr3 (28,) int32 and n_pairs3 (device int64). The caller turns row_cnt3 into row_ptr3 (n+1,
 * exclusive prefix sum) and, with the 5x5x5 lists of ptv3_kmap_plan_fill, _inner_fill writes pair_in3 /
 * pair_slot3 (allocate n_pairs5 entries: the 3x3x3 lists are never longer). */
int ptv3_kmap_plan_inner_count(const int32_t *tap_ptr5, int64_t n, const void *workspace5,
                               size_t workspace5_bytes, int32_t *found3, int32_t *row_cnt3,
                               int32_t *tap_ptr3, int64_t *n_pairs3, void *stream);
int ptv3_kmap_plan_inner_fill(const int32_t *tap_ptr5, const int32_t *row_ptr5, const int32_t *pair_in5,
                              const int32_t *pair_slot5, int64_t n, int64_t n_pairs5, const int32_t *found3,
                              const int32_t *tap_ptr3, const int32_t *row_ptr3, int32_t *pair_in3,
                              int32_t *pair_slot3, void *stream);
int ptv3_subm_conv_pairs_fwd(const void *feat, int dtype, int64_t n, int cin, int taps,
                             int64_t n_pairs, const int32_t *tap_ptr, const int32_t *row_ptr,
                             const int32_t *pair_in, const int32_t *pair_slot, const void *weight,
                             const void *bias, int cout, void *y, void *out, void *stream);

/* Tile form of the 3x3x3 convolution with cin == cout == channels in {64, 128} (the xCPE of
 * every block, model.py:546-552; ptv3_subm_conv_pack_weight itself takes any multiple of 32), fp16/bf16: a work-group keeps the fp32 sums of a tile of 128
 * consecutive output voxels on chip and walks their pairs tap by tap, so no product row per pair
 * goes through memory; sums in tap order, nothing atomic, same result on every run.
 * Lists, made once per plan (n < 2^24, taps == 27):
 *   ptv3_conv_plan_slots: the tap-major lists of a plan -> output-major words slot_pair (n_pairs,)
 *     int32, slot_pair[pair_slot[q]] = tap(q) << 24 | pair_in[q];
 *   ptv3_conv_plan_tiles: per tile its pairs sorted by tap. tile_tap (ptv3_conv_plan_tile_count(n),
 *     32) int32: [t] = first pair of tap t relative to the tile's first pair, [27] = pairs of the
 *     tile, [28] = the tile's first pair; tile_pair (n_pairs,) int32 = voxel inside the tile << 24 |
 *     input row (the order inside a tap is unspecified; no result depends on it).
 * ptv3_subm_conv_pack_weight stores the (channels, taps, channels) weight in MFMA fragment order
 * (same size); do it once per weight. */
int ptv3_conv_plan_slots(const int32_t *tap_ptr, int taps, const int32_t *pair_in, const int32_t *pair_slot,
                         int64_t n_pairs, int32_t *slot_pair, void *stream);
int64_t ptv3_conv_plan_tile_count(int64_t n);
int ptv3_conv_plan_tiles(const int32_t *row_ptr, const int32_t *slot_pair, int64_t n, int taps,
                         int32_t *tile_tap, int32_t *tile_pair, int32_t *vox_taps, void *stream);
int ptv3_subm_conv_pack_weight(const void *weight, int dtype, int channels, int taps, void *packed, void *stream);
/* ptv3_subm_conv_pack_weight for several weights in one launch (a model repacks all of them when its parameters
 * may have changed). The table lies in device memory; first_block is the running sum of
 * ptv3_subm_conv_pack_weight_blocks(channels, taps) over the jobs before this one, n_blocks the sum over all.
 * The table is trusted: channels must be a multiple of 32 and first_block that running sum. A row with other
 * channels is skipped by the kernel; a row whose buffers are smaller than (channels, taps, channels) is not
 * detected and writes out of bounds. */
typedef struct {
    const void *weight;   /* (channels, taps, channels), f16 or bf16 */
    void *packed;         /* same size and type */
    int32_t channels, taps;
    int64_t first_block;
} ptv3_pack_job;
int64_t ptv3_subm_conv_pack_weight_blocks(int channels, int taps);
int ptv3_subm_conv_pack_weight_batch(const ptv3_pack_job *jobs, int n_jobs, int64_t n_blocks, void *stream);
int ptv3_subm_conv_tiles_fwd(const void *feat, int dtype, int64_t n, int channels, int taps,
                             const void *packed_weight, const void *bias, const int32_t *tile_tap,
                             const int32_t *tile_pair, const int32_t *vox_taps, void *out, void *stream);
/* The same with tiles of tile_voxels outputs: 128 (what the three functions above use), or 96 at 128 channels
 * (same call site, model.py:546-552). The lists must have been made with the same tile_voxels. A launch runs in
 * rounds of the work-groups the part holds at a time; the caller picks the size whose last round is fuller. */
int64_t ptv3_conv_plan_tile_count_sized(int64_t n, int tile_voxels);
int ptv3_conv_plan_tiles_sized(const int32_t *row_ptr, const int32_t *slot_pair, int64_t n, int taps, int tile_voxels,
                               int32_t *tile_tap, int32_t *tile_pair, int32_t *vox_taps, void *stream);
int ptv3_subm_conv_tiles_fwd_sized(const void *feat, int dtype, int64_t n, int channels, int taps, int tile_voxels,
                                   const void *packed_weight, const void *bias, const int32_t *tile_tap,
                                   const int32_t *tile_pair, const int32_t *vox_taps, void *out, void *stream);

/* model.py:546-552 (spconv.SubMConv3d, 3x3x3, in == out channels) where a voxel has few neighbours: the same
 * tiles and packed weight as ptv3_subm_conv_tiles_fwd, but the work is in proportion to the pairs (an MFMA row
 * is a pair, not an output voxel with or without the tap) and nothing but feat, the lists and out touches
 * memory. channels 32 or 64; f16 / bf16. */
int ptv3_subm_conv_sparse_fwd(const void *feat, int dtype, int64_t n, int channels, int taps,
                              const void *packed_weight, const void *bias, const int32_t *tile_tap,
                              const int32_t *tile_pair, void *out, void *stream);

/* model.py:652-664,690-695: clusters of code0 >> shift walked in sorted order (order0 sorts
 * code0, so no further sort is needed). Outputs: cluster (n,) int64 [pooling_inverse],
 * indices (n,) int64 (= order0: points grouped by cluster), idx_ptr (n+1 allocated, m+1 used),
 * head (n allocated, m used), n_clusters (1 + n_scenes,) int64 on the device: the cluster count,
 * then (model.py:66-67 for the pooled point, without a bincount) the pooled cumulative scene ends
 * from the parent's offset (n_scenes,) int64 on the device; n_scenes may be 0 (offset unused). */
size_t ptv3_pool_clusters_workspace_bytes(int64_t n);
int ptv3_pool_clusters(const int64_t *code0, const int64_t *order0, int64_t n, int shift,
                       const int64_t *offset, int n_scenes, int64_t *cluster, int64_t *idx_ptr,
                       int64_t *head, int64_t *n_clusters, void *workspace, size_t workspace_bytes,
                       void *stream);

/* ptv3_pool_clusters for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. Same outputs as
 * ptv3_pool_clusters, bit for bit, and no workspace argument: the per-block cluster counts live in a fixed
 * 256 KiB array inside the library's device code, one copy per GPU, held until the process ends. Nothing is
 * allocated or freed, here or in a library underneath; the first call on a GPU looks the array's device
 * address up once (hipGetSymbolAddress): make that first call outside any graph capture, as a warm-up -- a
 * call with n = 0 does it and launches nothing. n <= ptv3_pool_clusters_static_max_points() = 16,777,216, else
 * PTV3_ESTATIC. The stream must belong to the current device. All calls on one GPU share the array: calls that
 * overlap on one GPU (two streams, or two threads) race on it and give wrong clusters -- serialise them; calls
 * on one stream are ordered. */
int64_t ptv3_pool_clusters_static_max_points(void);
int ptv3_pool_clusters_static(const int64_t *code0, const int64_t *order0, int64_t n, int shift,
                              const int64_t *offset, int n_scenes, int64_t *cluster, int64_t *idx_ptr,
                              int64_t *head, int64_t *n_clusters, void *stream);

/* model.py:666-674,690,695 once the cluster count m is known on the host: pooled codes
 * (k,m) = code[:, head] >> shift, pooled grid_coord (m,3) = grid_coord[head] >> pool_depth,
 * pooled batch (m,) = batch[head]; indices_out (m,4) int32 = [batch, x, y, z] of the pooled
 * points, the sparse tensor's indices (model.py:165-167), or NULL. row_perm: host array of k ints,
 * output row r is made from input row row_perm[r] (the shuffle of model.py:675-679 applied while
 * writing; k <= 16), or NULL for the identity. */
int ptv3_pool_gather(const int64_t *code, int64_t n, int k, int shift, const int32_t *grid_coord,
                     int pool_depth, const int64_t *batch, const int64_t *head, int64_t m,
                     const int32_t *row_perm, int64_t *code_out, int32_t *grid_coord_out,
                     int64_t *batch_out, int32_t *indices_out, void *stream);

/* model.py:667-674 without a sort: the pooled order of every curve is the sequence of distinct
 * clusters met when walking the parent points along that curve (order (k,n): the parent's
 * serialized_order; cluster (n,): pooling_inverse; m clusters). Writes order_out, inverse_out
 * (k,m) int64, identical to argsort of the pooled codes and its inverse. Requires what the
 * reference's pooling relies on too: a point's code shifted right is its cluster's code.
 * row_perm as for ptv3_pool_gather. */
size_t ptv3_pool_orders_workspace_bytes(int64_t n, int k);
int ptv3_pool_orders(const int64_t *order, const int64_t *cluster, int64_t n, int k, int64_t m,
                     const int32_t *row_perm, int64_t *order_out, int64_t *inverse_out, void *workspace,
                     size_t workspace_bytes, void *stream);

/* torch_scatter.segment_csr call sites model.py:684-689: reduce src[indices[j]] over
 * j in [idx_ptr[s], idx_ptr[s+1]). op 0 = max, 1 = mean, 2 = sum, 3 = min.
 * src (n,c) of dtype, out (m,c) of dtype. */
int ptv3_segment_reduce(const void *src, int dtype, int64_t n, int c, const int64_t *indices,
                        const int64_t *idx_ptr, int64_t m, int op, void *out, void *stream);

/* Weight gradient of nn.Linear (model.py:366-367, :505-507, :553, :633, :726-727 under autograd):
 * dweight[o][i] = sum over rows r of dout[r][o] * x[r][i]. x (n,k), dout (n,nout) fp16 / bf16 with k and
 * nout multiples of 8; dweight (nout,k) fp32, every element written; dbias (nout,) fp32 or NULL: the
 * column sums of dout, taken from the same pass over its rows. */
size_t ptv3_linear_wgrad_workspace_bytes(int64_t n, int k, int nout);
int ptv3_linear_wgrad(const void *x, const void *dout, int dtype, int64_t n, int k, int nout, float *dweight,
                      float *dbias, void *workspace, size_t workspace_bytes, void *stream);

/* The first Linear of the MLP with its GELU, for training (model.py:505-507: fc1, act): pre = x w^T + bias and
 * out = gelu(pre), both (n,nout) of dtype, from one pass; shapes as for ptv3_linear_fwd. */
int ptv3_linear_gelu_fwd(const void *x, const void *w, const void *bias, int dtype, int64_t n, int k, int nout,
                         void *pre, void *out, void *stream);

/* Input gradient of the second Linear of the MLP taken back through the GELU in front of it (model.py:506-507):
 * dpre = (dout wt^T) * gelu'(pre). dout (n,k) is the gradient of fc2's output, wt (nout,k) fc2's weight
 * transposed (hidden x out channels), pre (n,nout) as written by ptv3_linear_gelu_fwd, dpre (n,nout). */
int ptv3_linear_gelu_bwd(const void *dout, const void *wt, const void *pre, int dtype, int64_t n, int k, int nout,
                         void *dpre, void *stream);

/* Half-precision and transposed copies of fp32 master weights, many tensors per launch: what autocast does to the
 * weight of every nn.Linear / spconv.SubMConv3d (model.py:366-367, :505-507, :546-553, :767-774) on each use, and
 * the transposes their input gradients multiply by. One job per tensor; src is a contiguous fp32 (a, b, c) array.
 *   mirror = 0: dst[i] = src[i] for all a*b*c elements;
 *   mirror = 1: dst[(k*b + (b-1-j))*a + i] = src[(i*b + j)*c + k] -- (Cout, taps, Cin) to (Cin, mirrored taps, Cout);
 *               with b = 1 the plain transpose of a matrix.
 * first_block is the running sum of ptv3_cast_params_blocks(a, b, c, mirror) over the jobs before this one, and
 * n_blocks the sum over all jobs. The table itself lies in device memory, dst are of dst_dtype and must not
 * overlap any src. Shapes in the table are not checked: a wrong table writes out of bounds. */
typedef struct {
    const float *src;
    void *dst;
    int32_t a, b, c;
    int32_t mirror;
    int64_t first_block;
} ptv3_cast_job;
int64_t ptv3_cast_params_blocks(int a, int b, int c, int mirror);
int ptv3_cast_params(const ptv3_cast_job *jobs, int n_jobs, int64_t n_blocks, int dst_dtype, void *stream);

/* nn.LayerNorm for training (model.py:554, :557, :572), with the residual connection in front of it taken
 * into the same pass where there is one (model.py:589-604):
 * sum = skip + branch * row_scale, y = LayerNorm(sum). skip (n,c) and row_scale (n,) -- the stochastic-depth
 * factor per row, model.py:583 -- may be NULL; sum may be NULL when only y is wanted (then this is a plain
 * LayerNorm of branch). Every tensor has its own dtype code (0 fp32, 1 fp16, 2 bf16): under autocast the
 * residual stream is float and the branches half precision. gamma, beta (c,) of param_dtype.
 * c in {32, 64, 128, 256, 512}. The statistics are taken from sum as rounded to sum_dtype.
 * pre_gamma, pre_beta (c,) of param_dtype, both or neither NULL: the branch first goes through a LayerNorm of
 * its own (the xCPE's norm in front of a Block's first residual connection, model.py:546-554, :589-592),
 * sum = skip + LayerNorm_pre(branch) * row_scale, in the same pass and without rounding in between. */
int ptv3_add_layer_norm_fwd(const void *skip, int skip_dtype, const void *branch, int branch_dtype,
                            const void *row_scale, int row_scale_dtype, const void *gamma, const void *beta,
                            int param_dtype, int64_t n, int c, float eps, void *sum, int sum_dtype, void *y,
                            int y_dtype, const void *pre_gamma, const void *pre_beta, float pre_eps, void *stream);

/* Its backward: g = LayerNorm'(sum; dy) + dsum (dsum: the gradient that reaches sum past the LayerNorm, or
 * NULL); dskip = g and dbranch = g * row_scale, either may be NULL, each in its own dtype. dgamma, dbeta
 * (c,) fp32 are accumulated into (zero them first). With pre_x (the branch as the forward read it, n x c of
 * pre_x_dtype) the branch's own LayerNorm is taken back as well: dbranch is then the gradient of pre_x, and
 * dpre_gamma, dpre_beta (c,) fp32 are accumulated into like dgamma, dbeta. */
int ptv3_add_layer_norm_bwd(const void *sum, int sum_dtype, const void *dy, int dy_dtype, const void *dsum,
                            int dsum_dtype, const void *row_scale, int row_scale_dtype, const void *gamma,
                            int param_dtype, int64_t n, int c, float eps, void *dskip, int dskip_dtype,
                            void *dbranch, int dbranch_dtype, float *dgamma, float *dbeta, const void *pre_x,
                            int pre_x_dtype, const void *pre_gamma, float pre_eps, float *dpre_gamma,
                            float *dpre_beta, void *stream);

/* A residual connection with no LayerNorm behind it (model.py:602-604, the end of a Block, with the
 * stochastic-depth factor of model.py:583): out = skip + branch * row_scale, rows (n,c), c a multiple of 8, each
 * tensor in its own dtype. skip and row_scale (n,) may be NULL: with skip NULL this is the gradient of the
 * branch, dbranch = dout * row_scale, or a plain conversion. */
int ptv3_scaled_add(const void *skip, int skip_dtype, const void *branch, int branch_dtype, const void *row_scale,
                    int row_scale_dtype, int64_t n, int c, void *out, int out_dtype, void *stream);

/* nn.BatchNorm1d in training mode (model.py:848; call sites :776-779, :707-710, :729-735), first half: the
 * batch statistics of x (n,c), c in {32, 64, 128, 256, 512}. stats (3,c) fp32 receives mean, rsqrt(var + eps)
 * and the biased variance; running_mean / running_var (c,) fp32, when given, are updated in place with
 * `momentum` and the unbiased variance, as torch does. workspace: 2*c floats. The normalisation itself is
 * ptv3_bn_act with mean = stats[0], var = stats[2]. */
int ptv3_batch_norm_stats(const void *x, int dtype, int64_t n, int c, float eps, float momentum,
                          float *running_mean, float *running_var, float *stats, float *workspace,
                          void *stream);

/* Backward of BatchNorm1d, optionally through the exact GELU behind it (gelu != 0: dout is the gradient of
 * gelu(bn(x))). stats as written by ptv3_batch_norm_stats, or (running_mean, rsqrt(running_var + eps)) with
 * batch_stats = 0 for a module in evaluation mode. gamma, beta (c,) of param_dtype or NULL. dx (n,c) of
 * dx_dtype; dgamma_dbeta (2,c) fp32 receives the parameter gradients (every element written). */
int ptv3_batch_norm_bwd(const void *x, int x_dtype, const void *dout, int dout_dtype, const float *stats,
                        const void *gamma, const void *beta, int param_dtype, int64_t n, int c, int gelu,
                        int batch_stats, void *dx, int dx_dtype, float *dgamma_dbeta, void *stream);

/* Backward of ptv3_segment_reduce (torch_scatter.segment_csr's, model.py:684-689): dsrc (n,c).
 * max / min: the gradient of a cluster goes to the first member in list order whose value equals
 * out; sum: to every member; mean: divided by the cluster size. Every row of src must belong to
 * exactly one cluster (true for grid pooling), so every element of dsrc is written. */
int ptv3_segment_reduce_bwd(const void *src, const void *out, const void *dout, int dtype, int64_t n, int c,
                            const int64_t *indices, const int64_t *idx_ptr, int64_t m, int op, void *dsrc,
                            void *stream);

/* model.py:746: out[i] = parent[i] + child[cluster[i]]; parent,out (n,c), child (m,c). */
int ptv3_unpool_add(const void *parent, const void *child, int dtype, int64_t n, int c,
                    const int64_t *cluster, int64_t m, void *out, void *stream);

/* nn.LayerNorm calls model.py:554,557,572 fused with the residual adds :589,:594,:602.
 * x,res,out0,out1 (n,c); gamma,beta (c,); all of dtype, statistics in fp32.
 * mode 0: out0 = LN(x).  mode 1: out0 = res + LN(x).
 * mode 2: s = x + res, out1 = LN(s), out0 = s + shift (shift (c,) or NULL: the bias of a GEMM that
 *         will accumulate onto out0).
 * mode 3: out0 = res + LN(x), out1 = LN(out0) with the second affine pair gamma2,beta2.
 * Intermediates are rounded to dtype where separate kernels would have stored them. */
int ptv3_layer_norm(const void *x, const void *res, const void *gamma, const void *beta,
                    const void *gamma2, const void *beta2, const void *shift, int dtype, int64_t n,
                    int c, float eps, int mode, void *out0, void *out1, void *stream);

/* Inference-mode nn.BatchNorm1d (model.py:848) and the nn.GELU that follows it at model.py:776-779,
 * :707-710 and :729-735 in one pass: out = act((x - mean) * rsqrt(var + eps) * gamma + beta) per
 * channel; act 0 = none, 1 = exact GELU. x, out (n,c) of dtype; running_mean/var (c,) float32 when
 * stats_f32 != 0, else of dtype (a module cast with .half()); gamma, beta (c,) of dtype or NULL.
 * c % 8 == 0. */
int ptv3_bn_act(const void *x, const void *running_mean, const void *running_var, int stats_f32,
                const void *gamma, const void *beta, int dtype, int64_t n, int c, float eps, int act,
                void *out, void *stream);

/* nn.Linear of the wide blocks (model.py:541-545 cpe.1, :450 qkv, :487 proj, :510-512 fc1 + GELU):
 * out = act(x w^T + bias), x (n, k), w (nout, k), bias (nout,) or NULL, out (n, nout), act = exact
 * (erf) GELU when gelu != 0. fp16/bf16, k in {32, 64, 128, 256, 512}, nout a multiple of 32 (PTV3_ESHAPE
 * otherwise: ptv3_linear_any_fwd takes every shape). Tall-and-skinny form: rows held in MFMA operand registers, no loop
 * over memory along k. */
int ptv3_linear_fwd(const void *x, const void *w, const void *bias, int dtype, int64_t n, int k, int nout,
                    int gelu, void *out, void *stream);
/* The same layers at 256 inputs (the 16 cm level of the default model: cpe.1, qkv, proj, fc1 + GELU) with the
 * weights resident in registers instead of LDS: k == 256, nout a multiple of 256 (PTV3_ESHAPE otherwise: use
 * ptv3_linear_fwd). Same result as ptv3_linear_fwd: fp32 accumulation over the 256 inputs, one rounding. */
int ptv3_linear_wide_fwd(const void *x, const void *w, const void *bias, int dtype, int64_t n, int k, int nout,
                         int gelu, void *out, void *stream);
/* nn.Linear with a long contraction (model.py:514 fc2 of the wide blocks, 1024 -> 256 and 2048 -> 512, with the
 * residual addition of :602 taken in; :450 the 512 -> 1536 qkv): out = resid + x w^T + bias, a tiled GEMM.
 * x (n, k), w (nout, k), bias (nout,) or NULL, resid (n, nout) or NULL (it may be `out` itself: every element is
 * read before it is written, by the same thread), fp16 / bf16, k a multiple of 128, nout a multiple of 128
 * (PTV3_ESHAPE otherwise). Sums and the residual are added in fp32 and rounded once. */
int ptv3_linear_gemm_fwd(const void *x, const void *w, const void *bias, const void *resid, int dtype, int64_t n,
                         int k, int nout, void *out, void *stream);
/* nn.Linear of any shape (every call site above in an fp32 model, the reference's parity path with
 * enable_flash=False, model.py:458-474; half-precision layers whose widths the kernels above do not take):
 * out = resid + act(x w^T + bias), act = exact GELU when gelu != 0, resid (n, nout) or NULL (it may be `out`
 * itself: every element is read before it is written, by the same thread). fp32 / fp16 / bf16, any k and nout;
 * fp32 FMA arithmetic, one rounding. Not tuned: the MFMA kernels above take the shapes of the released models. */
int ptv3_linear_any_fwd(const void *x, const void *w, const void *bias, const void *resid, int dtype, int64_t n,
                        int k, int nout, int gelu, void *out, void *stream);
/* The same followed by an inference-mode nn.BatchNorm1d and optionally the GELU, the projections of
 * model.py:726-735 (Linear -> BatchNorm1d -> GELU) in one kernel; statistics and affine parameters as
 * for ptv3_bn_act. The Linear's result is rounded to dtype before the normalisation, as when stored. */
int ptv3_linear_bn_act_fwd(const void *x, const void *w, const void *bias, const void *running_mean,
                           const void *running_var, int stats_f32, const void *gamma, const void *beta,
                           float eps, int dtype, int64_t n, int k, int nout, int gelu, void *out, void *stream);
/* Square Linear (channels in and out, 128 or 256; fp16/bf16) fused with the LayerNorms and residual
 * additions that follow it in a block, semantics and rounding points of ptv3_layer_norm's modes with
 * x replaced by Linear(x):
 *   mode 2 (proj, model.py:487,594-597): s = res + Linear(x); out0 = s (+ shift); out1 = LN(s)
 *   mode 3 (cpe.1 + cpe.2, model.py:541-545,587-593): s = res + LN(Linear(x)); out0 = s; out1 = LN2(s)
 * w (channels, channels) as nn.Linear stores it, bias / shift (channels,) or NULL, gamma2 / beta2
 * for mode 3 only. */
int ptv3_linear_ln_fwd(const void *x, const void *w, const void *bias, const void *res, const void *gamma,
                       const void *beta, const void *gamma2, const void *beta2, const void *shift, int dtype,
                       int64_t n, int channels, int mode, float eps, void *out0, void *out1, void *stream);

/* MLP of a block plus its residual, model.py:510-516 and :602, in one kernel:
 * out = resid + fc2(GELU(fc1(x))), exact (erf) GELU, intermediates rounded to dtype where the
 * separate layers would have stored them. x, resid, out (n, channels); w1 (hidden, channels),
 * b1 (hidden,), w2 (channels, hidden), b2 (channels,). fp16/bf16, channels 32, 64, 128, 256 or
 * 512, hidden = 4 * channels (PTV3_ESHAPE otherwise: use the separate layers). */
int ptv3_mlp_fused(const void *x, const void *resid, const void *w1, const void *b1, const void *w2,
                   const void *b2, int dtype, int64_t n, int channels, int hidden, void *out,
                   void *stream);

/* The same MLP (model.py:510-516, :602) at 128, 256 or 512 channels with both weight matrices handed over in the
 * order the kernel streams them, so that every MFMA operand fragment is one contiguous KB (the layers' own
 * (out, in) layout costs the kernel 32 cache lines per load instruction). ptv3_mlp_pack_weights writes that
 * copy: packed holds 8 * channels^2 elements of dtype, first w1 (4 * channels, channels) and w2 (channels,
 * 4 * channels) interleaved chunk by chunk; redo it whenever the parameters change. Same results, bit for bit,
 * as ptv3_mlp_fused. */
int ptv3_mlp_pack_weights(const void *w1, const void *w2, int dtype, int channels, void *packed, void *stream);
/* The same packing for several MLPs in one launch (after an optimizer step every copy is stale at once): jobs is a
 * device array, first_block ascending from 0 with job j owning ptv3_mlp_pack_weights_blocks(channels) blocks,
 * n_blocks their sum. Both half types move as 16-bit patterns, so a table may mix them. The table is trusted like
 * ptv3_pack_job's: channels 128, 256 or 512 (other rows are skipped), buffers of the stated sizes. */
typedef struct {
    const void *w1, *w2;  /* (4 * channels, channels) and (channels, 4 * channels); w2 NULL: w1 is a */
    void *packed;         /* (k * channels, channels) matrix. 8 * channels^2 elements (k * channels^2 without w2) */
    int32_t channels, reserved;   /* reserved: k when w2 is NULL (0 counts as 1), else unused */
    int64_t first_block;
} ptv3_mlp_pack_job;
int64_t ptv3_mlp_pack_weights_blocks(int channels);
int ptv3_mlp_pack_weights_batch(const ptv3_mlp_pack_job *jobs, int n_jobs, int64_t n_blocks, void *stream);
int ptv3_mlp_fused_packed(const void *x, const void *resid, const void *packed, const void *b1, const void *b2,
                          int dtype, int64_t n, int channels, void *out, void *stream);

/* Second half of a block at 128 or 256 channels in one kernel, model.py:458-460 (proj), :595-602:
 *   sum = shortcut + (attn @ w_proj^T + b_proj)
 *   out = sum + fc2(GELU(fc1(LayerNorm_2(sum))))
 * attn, shortcut, out: (n, channels) of dtype (PTV3_F16 / PTV3_BF16); biases and LayerNorm parameters (channels) or
 * (4 * channels) of dtype. mlp_packed as for ptv3_mlp_fused_packed; proj_packed holds channels^2 elements, the
 * (channels, channels) weight in the same order: written by ptv3_mlp_pack_weights_batch from a job whose w2 is NULL
 * (w1 = the weight, packed = proj_packed), which owns ptv3_linear_pack_weights_blocks(channels) blocks of the launch.
 * The projection, the sum and the normalised rows are rounded to dtype where the separate layers would store them
 * and never leave the CU. PTV3_ESHAPE for other widths or dtypes. */
int64_t ptv3_linear_pack_weights_blocks(int channels);

/* First half of a block behind its convolution at 128 or 256 channels in one kernel, model.py:541-545 (the xCPE's
 * Linear and LayerNorm), :587-589, :592-593 (norm1) and :450 (qkv):
 *   feat = shortcut + LayerNorm_cpe(conv @ w_cpe^T + b_cpe)
 *   qkv  = LayerNorm_1(feat) @ w_qkv^T + b_qkv
 * conv, shortcut, feat: (n, channels) of dtype; qkv: (n, 3 * channels). packed holds 4 * channels^2 elements: w_cpe
 * (channels, channels) and behind it w_qkv (3 * channels, channels), each written by ptv3_mlp_pack_weights_batch from
 * a job whose w2 is NULL and whose `reserved` is the number of channels-row chunks (1 and 3; packed = the buffer, and
 * the buffer + channels^2 elements); such a job owns reserved * ptv3_linear_pack_weights_blocks(channels) blocks.
 * Intermediates are rounded to dtype where the separate layers would store them; the normalised rows never leave
 * the CU. PTV3_ESHAPE for other widths or dtypes. */
int ptv3_block_head_wide(const void *conv, const void *shortcut, const void *packed, const void *cpe_bias,
                         const void *ln_cpe_weight, const void *ln_cpe_bias, float ln_cpe_eps, const void *ln1_weight,
                         const void *ln1_bias, float ln1_eps, const void *qkv_bias, int dtype, int64_t n, int channels,
                         void *feat, void *qkv, void *stream);
int ptv3_block_tail_wide(const void *attn, const void *shortcut, const void *proj_packed, const void *proj_bias,
                         const void *ln_weight, const void *ln_bias, float ln_eps, const void *mlp_packed,
                         const void *b1, const void *b2, int dtype, int64_t n, int channels, void *out, void *stream);

/* Head of a block for thin channels, model.py:541-545, :587-589, :592-593 and :450 in one kernel:
 *   feat = shortcut + LayerNorm_cpe(conv @ w_cpe^T + b_cpe)
 *   qkv  = LayerNorm_1(feat) @ w_qkv^T + b_qkv
 * (cpe.1, cpe.2, the residual, norm1 and attn.qkv), intermediates rounded to dtype where the
 * separate layers would have stored them. conv, shortcut, feat (n, channels); qkv (n, 3*channels);
 * w_cpe (channels, channels); w_qkv (3*channels, channels); biases and LayerNorm parameters of
 * dtype, NULL = 0 (bias, beta) or 1 (gamma). fp16/bf16, channels 32 or 64 (PTV3_ESHAPE otherwise:
 * use the separate layers). */
int ptv3_block_head_fused(const void *conv, const void *shortcut, const void *w_cpe, const void *b_cpe,
                          const void *ln_cpe_gamma, const void *ln_cpe_beta, float ln_cpe_eps,
                          const void *ln1_gamma, const void *ln1_beta, float ln1_eps, const void *w_qkv,
                          const void *b_qkv, int dtype, int64_t n, int channels, void *feat, void *qkv,
                          void *stream);

/* Tail of a block for thin channels, model.py:485-487, :594-595 and :599-602 in one kernel:
 *   feat = shortcut + (attn @ w_proj^T + b_proj)
 *   out  = feat + fc2(GELU(fc1(LayerNorm_2(feat))))
 * (attn.proj, the residual, norm2, the MLP and its residual; exact GELU), rounded like the separate
 * layers. attn, shortcut, out (n, channels); w_proj (channels, channels); w1 (hidden, channels);
 * w2 (channels, hidden); fp16/bf16, channels 32 or 64, hidden = 4 * channels. */
int ptv3_block_tail_fused(const void *attn, const void *shortcut, const void *w_proj, const void *b_proj,
                          const void *ln2_gamma, const void *ln2_beta, float ln2_eps, const void *w1,
                          const void *b1, const void *w2, const void *b2, int dtype, int64_t n,
                          int channels, int hidden, void *out, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PTV3_HIP_H */
