/*
 * glowq_w4a16.h - C ABI of the MI355X (gfx950) implementation of GlowQ's Step-3 inference hot
 * path: the W4A16 quantised linear (int4 codes packed 8 per int32, asymmetric per-group scale and
 * zero-point, fp16 activations) fused with the group-shared low-rank correction.
 *
 * All pointers are DEVICE pointers unless stated otherwise.  fp16 tensors are passed as
 * `const void*` (IEEE binary16, row-major).  Every entry point launches asynchronously on
 * `stream` (a hipStream_t passed as void*; NULL = the default stream), never synchronises and never
 * allocates.  Return value: GLOWQ_OK (0) or a negative GLOWQ_E* code; `glowq_last_error()` returns
 * the message of the calling thread's last failure.
 *
 * Tensor conventions (identical to the reference's buffers, src/cuda_w4a16/linear.py:104-106):
 *   x        [M, K]            fp16, row stride K
 *   qweight  [N, ldw_i32]      int32, element k of row n is nibble (k & 7) of word (k >> 3)
 *   scales   [N, lds]          fp16, one per group of `group_size` input columns
 *   qzeros   [N, ldz_i32]      int32, zero-point of group g is nibble (g & 7) of word (g >> 3)
 *   y        [M, N]            fp16, row stride ldy
 * Naming of the low-rank factors: R is the shared right factor [rank, K] (the reference's
 * `B_shared` / wrapper argument `B_q`); L is a module's left factor [N, rank] (the reference's
 * `{group}.{module}.A` / wrapper argument `A_q`), src/step3_eval_dataset.py:484,506.
 */
#ifndef GLOWQ_W4A16_H_
#define GLOWQ_W4A16_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GLOWQ_OK 0
#define GLOWQ_EINVAL (-1)     /* bad argument (null pointer, non-positive size, bad group_size) */
#define GLOWQ_ESHAPE (-2)     /* leading dimensions too small for the stated shape */
#define GLOWQ_ELAUNCH (-3)    /* the HIP runtime reported a launch error */
#define GLOWQ_EUNSUPPORTED (-4)

#define GLOWQ_MAX_MEMBERS 4

/* One module of a QKV / MLP group (q, k, v or gate, up), or a solo module (o_proj, down_proj). */
typedef struct glowq_member {
  const int32_t* qweight; /* [N, ldw_i32] */
  const void* scales;     /* [N, lds] fp16 */
  const int32_t* qzeros;  /* [N, ldz_i32] */
  const void* L;          /* [N, rank] fp16 left factor, or NULL: no correction (GlowQ-S unselected) */
  const void* bias;       /* [N] fp16 or NULL */
  void* y;                /* [M, N] fp16 output, row stride ldy */
  int32_t N;
  int32_t ldw_i32;
  int32_t lds;
  int32_t ldz_i32;
  int32_t ldy;
  int32_t side_rank;      /* the rank `side` was packed for (0: packed without a left factor) */
  const void* side;       /* the member's side stream written by glowq_pack_side for this K and group_size, or NULL */
  const void* tiled;      /* the member's tiled weights written by glowq_pack_tiled for this K and group_size, or NULL */
  const void* tiled_L;    /* its tiled left factor written by glowq_pack_tiled_left for tiled_rank, or NULL */
  int32_t tiled_rank;
  int32_t reserved;
} glowq_member_t;

/* Library / device information. */
int glowq_version(void);
const char* glowq_last_error(void);

/*
 * y = fp16( sum_k (code - zero) * scale * x ), fp32 accumulate.
 * Replaces `w4a16_gemv_forward_cuda` (src/cuda_w4a16/csrc/gemv_w4a16.cu:146-214; pybind
 * src/cuda_w4a16/csrc/pybind.cpp:19-23).  Any M is accepted; all M rows share one pass over the weights.
 * Weight rounding by row count: the GEMV kernels (1 token row; 2..4 rows by group size, see glowq_set_tuning) keep
 * (code - zero) * scale unrounded, as the reference's GEMV does (gemv_w4a16.cu:96-112), and so does the raw-code
 * form of the skinny MFMA kernel (route 7: 5..8 rows by default, where K is a multiple of 256 and the groups have 128
 * columns).  On the other MFMA routes (1 and 2, glowq_w4a16_route tells) the dequantised weight is rounded once to fp16
 * before the multiply, which is the arithmetic of the reference's dequantise-then-matmul route (gemm_w4a16.cu:46-49,132)
 * -- the reference itself switches to that arithmetic only above 128 rows.  On activations of order one the two differ
 * by far less than 1e-2 + 1e-3 |y|; with outlier channels in the thousands they differ by more than that, in the
 * reference as here, so compare against the matching one.  glowq_set_tuning("quad_max_m", 16) together with
 * ("small_group_mb", 0) keeps the unrounded arithmetic (the 4x4x4 GEMV) up to 16 rows.
 */
int glowq_w4a16_gemv_forward(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                             void* y, int M, int K, int N, int group_size, int ldw_i32, int lds, int ldz_i32,
                             void* stream);

/*
 * Same contract for the large-M route: replaces `w4a16_gemm_forward_cuda`
 * (src/cuda_w4a16/csrc/gemm_w4a16.cu:76-135; pybind src/cuda_w4a16/csrc/pybind.cpp:24-27).  The
 * reference dequantises the whole weight to fp16 in HBM and calls a library GEMM; here the int4 codes
 * are dequantised on the fly ( fp16((code - zero) * scale), the same single rounding ) and fed to
 * fp16 MFMA with fp32 accumulate.  `split_k_iters` is accepted and ignored, as in the reference
 * (gemm_w4a16.cu:83).
 */
int glowq_w4a16_gemm_forward(const void* x, const int32_t* qweight, const void* scales, const int32_t* qzeros,
                             void* y, int M, int K, int N, int group_size, int split_k_iters, int ldw_i32,
                             int lds, int ldz_i32, void* stream);

/*
 * out[n, k] = fp16( (code - zero) * scale ), out is [N, K] with row stride K.  Replaces
 * `dequant_w4a16_asym_i32_kernel` (src/cuda_w4a16/csrc/gemm_w4a16.cu:19-50) and is the device twin of
 * `CudaW4A16Linear._dequant_chunk` (src/cuda_w4a16/linear.py:248-253).
 */
int glowq_w4a16_dequant(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* out, int N, int K,
                        int group_size, int ldw_i32, int lds, int ldz_i32, void* stream);

/*
 * codes[n, k] = nibble (k & 7) of word (k >> 3), as uint8.  Device twin of `_unpack_int4_i32`
 * (src/cuda_w4a16/linear.py:49-54; device form src/cuda_w4a16/csrc/gemv_w4a16.cu:16-25).
 */
int glowq_unpack_int4(const int32_t* packed, uint8_t* codes, int rows, int total_vals, int ld_i32, void* stream);

/*
 * r[m, j] = fp16( sum_k x[m, k] * R[j, k] ): the shared right-factor projection, computed once per
 * group and reused by every member.  Replaces `F.linear(x, B_q)` in `AddSVDCorrection.forward`
 * (src/step3_eval_dataset.py:484,497,501,504).  r is [M, rank], row stride rank.
 */
int glowq_shared_proj(const void* x, const void* R, void* r, int M, int K, int rank, void* stream);

/*
 * The same with a caller-provided workspace (same reference lines).  With more than 16 token rows (more than 64, or
 * M * K * rank above 90 million, from where the MFMA projection is used) the output [M, rank] is too small to fill the chip, so K is split over workgroups that leave fp32 partial tiles in `workspace`; a second
 * small launch adds them in slice order (results do not depend on scheduling) and writes r.
 * `workspace`: 16-byte aligned device memory, contents irrelevant; glowq_proj_workspace_bytes gives the size that lets
 * the split go as far as it is useful for a shape -- a smaller one splits less, NULL or 0 bytes is glowq_shared_proj.
 * Calls that share a workspace must not overlap (one workspace per stream).
 */
int glowq_shared_proj_ws(const void* x, const void* R, void* r, int M, int K, int rank, void* workspace,
                         size_t workspace_bytes, void* stream);
size_t glowq_proj_workspace_bytes(int M, int K, int rank);

/*
 * Side stream of a member: its scales, zero-points and left-factor rows (L may be NULL) repacked, two output rows at a
 * time, into the order the single-token decode GEMV consumes them in, so that a wave fetches them with one to three
 * coalesced loads per row block instead of a small request per array and row.  A deterministic function of the
 * canonical buffers, which stay what every other kernel reads (the reference has no counterpart: its GEMV reads
 * scale and zero-point per thread and row, src/cuda_w4a16/csrc/gemv_w4a16.cu:96-104).  glowq_side_bytes gives the
 * size of `side` (16-byte aligned device memory), 0 for shapes the layout does not cover (K a multiple of 32 up to
 * 18432, power-of-two groups of 128 columns and more, even ranks up to 256).  A member whose `side` is set must have
 * been packed for the K and group_size of the call and with the same L, and states the rank it was packed for in
 * `side_rank`; single-token calls read it instead of scales / qzeros / L when every member of the group brings one
 * whose rank is the rank the call applies (0 for a call without correction), and ignore it otherwise.
 */
size_t glowq_side_bytes(int N, int K, int group_size, int rank);
int glowq_pack_side(const void* scales, const int32_t* qzeros, const void* L, void* side, int N, int K, int group_size,
                    int rank, int lds, int ldz_i32, void* stream);

/*
 * One launch for a whole group: for every member i
 *     y_i = fp16( W4A16(x; member i) + bias_i + alpha * r @ L_i^T )
 * with r = the [M, rank] fp16 result of glowq_shared_proj (may be NULL when no member has L).
 * Members with L == NULL get no correction (the GlowQ-S selective path).  Replaces, per member, the
 * sequence inner(x) -> F.linear(r, A_q) -> z.add_(svd_raw, alpha) of `AddSVDCorrection.forward`
 * (src/step3_eval_dataset.py:470-511) and the selective wrapping of
 * `patch_svd_correction_wrappers_cumulative` (src/restoration/step4_evaluate_cumulative.py:99-154).
 * `members` is a HOST pointer to `n_members` (1..GLOWQ_MAX_MEMBERS) descriptors; it is copied
 * into the launch and may be reused as soon as the call returns.
 */
int glowq_w4a16_group_forward(const void* x, const void* r, const glowq_member_t* members, int n_members, int M,
                              int K, int group_size, int rank, float alpha, void* stream);

/*
 * Projection and group in one call: r_out = fp16(x R^T) ([M, rank], for the caller's group cache) followed by
 * the group launch that consumes it.  Replaces the whole body of `AddSVDCorrection.forward` for a group
 * (src/step3_eval_dataset.py:470-511) with one library call (two launches on `stream`; one where the variant with a
 * workspace below can compute r inside the group launch).
 */
int glowq_w4a16_group_forward_fused(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                    int n_members, int M, int K, int group_size, int rank, float alpha, void* stream);
/*
 * The two group entry points with a workspace (16-byte aligned device memory, contents irrelevant, not shared by calls
 * that overlap).  It serves the many-row projection as in glowq_shared_proj_ws and, on the tiled GEMM route, a split of
 * K where the output has too few tiles to fill the chip (long K, few columns: o_proj / down_proj at some hundred
 * rows): partial fp32 tiles, added in slice order by a second launch.  A slice of the split takes
 * 4 * roundup(M, 128) * sum_i roundup(N_i, 256) bytes; the split goes as far as the workspace holds slices.
 * The skinny MFMA route (5..64 rows) splits K the same way where its column tiles cover half of the CUs or fewer and
 * K is 12288 columns or longer (down_proj): 4 * M * sum_i roundup(N_i, 32) bytes per slice, at most 8 slices.
 * With a workspace of 6144 bytes or more, a fused call with one token row on the stream GEMV (route 5, ranks up to 256)
 * computes r inside the group launch where the whole grid of that launch is on the chip at once: workgroups in front
 * of the grid produce the entries of r, write them to r_out and hand them to the others through tagged words in the
 * workspace (the first 6144 bytes; the tags name the launch, so the words need no clearing and a replay of a captured
 * graph is a launch like any other).  One launch instead of two, the same bits in r_out and in the outputs as the
 * projection launch in front gives; "proj_in_launch" of glowq_set_tuning switches it off.  As everywhere, calls that
 * share a workspace must not overlap.
 * The skinny MFMA route does the same at 2..32 token rows where its launch leaves enough compute units free for the
 * workgroups that produce r (a workgroup per one or two blocks of four token rows by four rows of R; every group of an 8B
 * layer at 8 and 16 rows): they write r_out with stores that pass the caches private to a part of the chip and raise a
 * tagged flag each, the first of them turns the flags into one ready word, and the waves that apply the correction -- behind
 * their weights instead of in front of them -- read r_out once they see that word.  The head of the workspace (8192
 * bytes) holds flags and ready word, the partial tiles of a split of K lie behind it.  Outputs agree with the
 * two-launch form to rounding (the correction is added last instead of first), r_out in the arithmetic of the small
 * projection kernels.  A launch that computes r itself is not cut into two slices of K (down_proj of an 8B layer: one
 * launch instead of three).  A fused call with three or four token rows and such a workspace takes this kernel too where
 * its launch computes r itself (q|k|v, o_proj, down_proj; "small_rows_in_launch" of glowq_set_tuning switches that off),
 * instead of the projection launch and the launch of the 2..4-row kernels.
 * The kernel that streams the tiled copy does it at 5..16 token rows and ranks up to 256 where its grid is not cut into
 * slices of K and leaves compute units free (gate|up): producers in front as above, and the waves that stage the
 * activations of each workgroup look for the ready word when r is due in the stages, behind the last columns of K.  Same
 * 8192 bytes at the head of the workspace; the same bits in r_out and in the outputs as the two-launch form.
 */
int glowq_w4a16_group_forward_ws(const void* x, const void* r, const glowq_member_t* members, int n_members, int M,
                                 int K, int group_size, int rank, float alpha, void* workspace, size_t workspace_bytes,
                                 void* stream);
int glowq_w4a16_group_forward_fused_ws(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                       int n_members, int M, int K, int group_size, int rank, float alpha,
                                       void* workspace, size_t workspace_bytes, void* stream);

/*
 * Tiled copy of a member's weights for the matrix-core routes (5..64 token rows, from 2 on groups of 80 MB of codes and more): the codes of 32 output rows and 256
 * input columns at a time in the order in which one coalesced 16-byte-per-lane load hands every lane the B operand of
 * the 32x32x16 matrix instruction, with each lane's scale and -(1024 + zero-point) behind them (4352 bytes per
 * (row block, super-block); layout in glowq_amd/csrc/tiled.hpp).  A deterministic function of the canonical buffers,
 * which stay the state-dict form and what every other route reads; the reference has no counterpart (its large-M
 * route writes a dequantised fp16 copy of the whole weight on every call, src/cuda_w4a16/csrc/gemm_w4a16.cu:106-129).
 * glowq_tiled_bytes / glowq_tiled_left_bytes give the sizes (16-byte aligned device memory), 0 where the layout does not
 * apply (it needs K % 256 == 0 and power-of-two groups of 128 columns and more; ranks that are multiples of 8).
 * A member whose `tiled` is set must have been packed for the K and group_size of the call; `tiled_L` for its L and
 * `tiled_rank`.  Calls use them when every member of the group brings them, and ignore them otherwise.
 */
size_t glowq_tiled_bytes(int N, int K, int group_size);
int glowq_pack_tiled(const int32_t* qweight, const void* scales, const int32_t* qzeros, void* tiled, int N, int K,
                     int group_size, int ldw_i32, int lds, int ldz_i32, void* stream);
size_t glowq_tiled_left_bytes(int N, int rank);
int glowq_pack_tiled_left(const void* L, void* tiled_L, int N, int rank, void* stream);

/*
 * glowq_w4a16_group_forward_fused_ws for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and results as
 * glowq_w4a16_group_forward_fused_ws called with a workspace of glowq_static_scratch_bytes() bytes, but the workspace
 * is a static device array inside the library (8 MiB on every GPU the library runs on, held until the process ends);
 * the call allocates and frees nothing.  At most GLOWQ_STATIC_MAX_ROWS token rows, and shapes whose projection would
 * want a larger workspace (glowq_proj_workspace_bytes) are refused with GLOWQ_EUNSUPPORTED.  Every call on a GPU shares
 * that GPU's array: calls that overlap on one GPU (two streams, two threads) race; nothing in it has to start at zero.
 * The first use on a device looks the array's address up (a symbol lookup, possibly a lazy load of the code object):
 * a caller that records the entry point into a graph calls glowq_static_scratch_prepare() on that device beforehand,
 * outside the capture; a call on a capturing stream of a device that was never prepared is refused with
 * GLOWQ_EUNSUPPORTED instead of doing that lookup under capture.
 */
#define GLOWQ_STATIC_MAX_ROWS 64
int glowq_w4a16_group_forward_fused_static(const void* x, const void* R, void* r_out, const glowq_member_t* members,
                                           int n_members, int M, int K, int group_size, int rank, float alpha,
                                           void* stream);
size_t glowq_static_scratch_bytes(void);
/* Resolves the static scratch of the current device (idempotent, allocates nothing); GLOWQ_OK or GLOWQ_ELAUNCH. */
int glowq_static_scratch_prepare(void);

/*
 * Kernel route chosen for a given row count, for reporting: 0 = wave-dot GEMV, 1 = skinny MFMA,
 * 2 = tiled MFMA GEMM, 3 = generic (odd shapes), 4 = 4x4x4 matrix-core GEMV, 5 = stream GEMV (every request of a
 * wave in flight up front; the default at one token row), 6 = the 4x4x4 matrix-core GEMV under the stream GEMV's
 * memory schedule (the default at two to four token rows), 7 = skinny MFMA with the int4 codes fed to the matrix
 * cores as they are and scale and zero-point applied to each group's sum (unrounded arithmetic; the default at five to
 * eight token rows).
 */
int glowq_w4a16_route(int M, int K, int N, int group_size, int ldw_i32);
/* The same for a member that brings the tiled copy of its weights (glowq_pack_tiled): 8 = the matrix-core kernel that
 * streams the tiled copy: 33..64 token rows, and 5..32 where the group's codes are 40 MB and more (24 MB from 17 rows);
 * "tiled_min_m" / "tiled_max_m" / "tiled_shape_rule" of glowq_set_tuning. */
int glowq_w4a16_route_tiled(int M, int K, int N, int group_size, int ldw_i32);

/*
 * Measurement helpers of bench.py; no counterpart in the reference.
 * glowq_last_launch: what the calling thread's last group launch used -- the kernel with the template arguments of the
 *   instantiation where the launcher records them (the stream GEMV, the tiled-copy kernel), else the route's name --
 *   and its grid and workgroup size (0 where not recorded).
 * glowq_probe_stream_read: a kernel that does nothing but read `bytes` (16-byte loads, eight in flight per lane,
 *   workgroup b the b-th contiguous share) with the given grid and workgroup size: the rate a memory-bound kernel of
 *   that launch shape could reach with no arithmetic at all.  `sink` (4 bytes of device memory) is never written.
 * glowq_probe_empty_launch: a kernel of that launch shape that returns at once (back-to-back launch cost).
 */
int glowq_last_launch(char* kernel, size_t bytes, int* grid_x, int* grid_y, int* block);
int glowq_probe_stream_read(const void* src, size_t bytes, void* sink, int grid, int block, void* stream);
int glowq_probe_empty_launch(int grid, int block, void* stream);

/*
 * Route limits of the process (the reference's counterpart is the W4A16_GEMV_M_MAX family of environment
 * knobs, src/cuda_w4a16/linear.py:21-27,122): "quad_max_m" / "quad_min_m" bound the token rows served by the
 * 4x4x4 matrix-core GEMV (0 for quad_max_m switches it off), "wave_dot_max_m" those of the wave-dot GEMV,
 * "skinny_max_m" (at most 64) those of the skinny MFMA kernel, above which the tiled GEMM takes over.
 * "small_group_mb": at 3..4 token rows a group whose int4 weights are smaller than this many MB goes to the
 * skinny MFMA kernel (or stays on the wave-dot GEMV) instead of the 4x4x4 GEMV, which starts up more slowly; at 2
 * rows it stays on the wave-dot GEMV and the limit is 40/17 of it; 0 = never.
 * "stream_max_m" (0..4): token rows up to which the stream GEMV is used where its layout applies, ahead of the
 * others; 0 switches it off.  "stream_shape_rule" (0 / 1): with more than one token row, only for the shapes it was
 * measured faster on (1, the default) or for every shape (0).
 * "qstream_max_m" (0..4, default 4): token rows, from two, up to which the stream-scheduled 4x4x4 matrix-core GEMV
 * is used where it applies (groups of 128 to 2048 columns, rank a multiple of 8 up to 128 or of 16 up to 256, rows
 * up to 16384 columns), ahead of all others; 0 switches it off.  "qstream_shape_rule" (0 / 1): only for the shapes it
 * was measured faster on (1, the default) or for every shape it can take (0).
 * "skinny_codes_max_m" (0..64, default 8): token rows up to which the skinny MFMA kernel runs in its raw-code form
 * (route 7) where that applies; above it is slower than dequantising first (the work on the sums grows with the rows).
 * "tiled_min_m" / "tiled_max_m" (default 2 / 64; max 0 switches the route off): token rows served by the kernel that
 * streams the tiled copy of the weights where every member brings one; "tiled_shape_rule" (0 / 1): up to 32 rows only
 * for groups whose stream is long enough to pay for its start-up (1, the default: 80 MB of codes up to 4 rows, 40 MB up to
 * 16, 24 MB up to 32) or for every group (0).
 * "proj_in_launch" (0 / 1, default 1): a fused single-token call with a workspace computes r inside the group launch
 * where that applies (glowq_w4a16_group_forward_fused_ws); 2, for tests, keeps the producing waves from handing their
 * entries over, so that every reader runs into "proj_spin_limit" (default 16384, 0 = never waits: the number of times
 * a reader looks again for an entry of r that is not there yet before it computes the entry itself).
 * Returns the previous value (>= 0) or GLOWQ_EINVAL.  Initial values come from GLOWQ_QUAD_M,
 * GLOWQ_QUAD_MIN_M, GLOWQ_WAVEDOT_M, GLOWQ_SKINNY_M, GLOWQ_SMALL_GROUP_MB, GLOWQ_STREAM_M, GLOWQ_STREAM_SHAPE_RULE,
 * GLOWQ_QSTREAM_M, GLOWQ_QSTREAM_SHAPE_RULE, GLOWQ_SKINNY_CODES_M, GLOWQ_TILED_MIN_M, GLOWQ_TILED_MAX_M,
 * GLOWQ_TILED_SHAPE_RULE, GLOWQ_PROJ_IN_LAUNCH and GLOWQ_PROJ_SPIN_LIMIT.
 */
int glowq_set_tuning(const char* key, int value);

/*
 * ---- single-token decode step around the linears --------------------------------------------------------
 * The reference runs these through Hugging Face's LlamaDecoderLayer (transformers, not vendored; its generate()
 * loop is what `measure_generation_metrics` times, src/step3_eval_dataset.py:705-798, and the manual KV-cache loop
 * of test/step3_1_layerwise.py:181-210).  Here they are four launches per layer that a HIP graph can replay.
 * All tensors fp16 unless typed otherwise; positions and tokens are int64 on the device.
 */

/* x[m] += delta[m] (skipped when delta is NULL), h[m] = rmsnorm(x[m]) * weight; x [M, H] is updated in place. */
int glowq_add_rmsnorm(void* x, const void* delta, const void* weight, void* h, int M, int H, float eps, void* stream);

/* out = silu(gate) * up over n elements (n % 8 == 0). */
int glowq_silu_mul(const void* gate, const void* up, void* out, long n, void* stream);

/*
 * The two above for one token, each also writing r = (its output) R^T ([rank] fp16, R [rank, H] resp. [rank, n]) for the
 * group launch that consumes the output: one launch instead of two.  x_out must not alias x_in.
 */
int glowq_add_rmsnorm_proj(const void* x_in, const void* delta, const void* weight, void* x_out, void* h, const void* R,
                           void* r, int H, int rank, float eps, void* stream);
int glowq_silu_mul_proj(const void* gate, const void* up, void* out, const void* R, void* r, int n, int rank, void* stream);

/*
 * Rotary embedding of q [heads, d] and k_new [kv_heads, d] at position *pos (cos/sin tables [max_len, d] fp32),
 * append of k / v_new to the caches [kv_heads, max_len, d] at *pos, attention of the one query token over positions
 * 0..*pos, out [heads, d].  d = 64 or 128; one pass with a running maximum, so max_len is bounded by the caches alone.
 * *pos is read on the device: a value outside [0, max_len) makes the launch write nothing at all (no cache row, no
 * output, no partial), so a replayed graph that steps past the end of the cache cannot write out of bounds.
 */
int glowq_rope_attend(const void* q, const void* k_new, const void* v_new, const float* cos_table, const float* sin_table,
                      const int64_t* pos, void* cache_k, void* cache_v, void* out, int heads, int kv_heads, int head_dim,
                      int max_len, float scale, void* stream);

/*
 * The same with the cached positions dealt row by row to `splits` workgroups per head: each writes its unnormalised
 * partial {max, sum, 2 unused, acc[d]} to partials [heads, splits, d + 4] fp32 (caller's buffer).  glowq_attend_combine_proj merges them
 * into out [heads * d] fp16 and, when R [rank, heads * d] is given, also writes r = out R^T ([rank] fp16) for the group
 * that consumes the attention output -- the o_proj group then needs no projection launch.
 */
int glowq_rope_attend_split(const void* q, const void* k_new, const void* v_new, const float* cos_table, const float* sin_table,
                            const int64_t* pos, void* cache_k, void* cache_v, float* partials, int splits, int heads,
                            int kv_heads, int head_dim, int max_len, float scale, void* stream);
int glowq_attend_combine_proj(const float* partials, void* out, const void* R, void* r, int heads, int head_dim, int splits,
                              int rank, void* stream);

/*
 * ---- chained group launches (single token) --------------------------------------------------------------
 * The work between two linears of a decoder layer -- residual add, RMSNorm or SwiGLU gate, and the projection of the
 * result on the next group's right factor -- done inside the two group launches on either side of it, so that a
 * layer is q|k|v, attention, merge, o_proj, gate|up, down_proj: six launches, none of them a norm, a gate or a
 * projection.  The modules the reference runs there are Hugging Face's LlamaRMSNorm, the residual adds and LlamaMLP's
 * act_fn(gate) * up around the wrappers' forward (src/step3_eval_dataset.py:470-511, generate loop :705-798); results
 * agree with the separate launches above within fp16 rounding of r (the projection is taken of the unrounded norm).
 *
 * prologue  GLOWQ_CHAIN_PRO_PLAIN     x [K] and r [rank] as in glowq_w4a16_group_forward
 *           GLOWQ_CHAIN_PRO_ACC       x [K] as given, r = fp16(P) with P read from acc_in
 *           GLOWQ_CHAIN_PRO_NORM_ACC  x is the residual stream [K]: the launch applies RMSNorm(norm_weight, eps) to it
 *                                     itself and takes r = fp16(f P), f the norm's scalar factor
 * epilogue  GLOWQ_CHAIN_EPI_NONE      outputs to the members' y
 *           GLOWQ_CHAIN_EPI_RESIDUAL  one member: resid[n] = fp16(resid[n] + y[n]) in place (y itself is written only
 *                                     if the member's y is not NULL); with next_Rt: P = next_R (next_norm_weight (.) resid)
 *                                     added into acc_out (next_norm_weight NULL: all ones)
 *           GLOWQ_CHAIN_EPI_SWIGLU    two members of equal N (gate, up): act[n] = fp16(fp16(silu(gate[n])) * up[n]);
 *                                     with next_Rt: P = next_R act added into acc_out
 * Served combinations: (NORM_ACC, NONE), (NORM_ACC, SWIGLU), (PLAIN, SWIGLU), (PLAIN, RESIDUAL), (ACC, RESIDUAL).
 * next_Rt is the next group's right factor transposed, [N_total, rank] fp16 row-major, of the same rank as this launch.
 * An accumulator is GLOWQ_CHAIN_ACC_BYTES of device memory, 8-byte aligned, all zero when the producer starts (the
 * caller clears it once per token, e.g. with a fill kernel; 64-bit fixed-point sums, so results do not depend on the
 * order in which workgroups finish).  A partial sum too large for the fixed point (|.| >= 2^31 / workgroups) or NaN
 * makes the consumer's r NaN rather than wrong.  Chained prologues and epilogues need rank > 0, L on every member and
 * a shape the stream GEMV takes (K % 32 == 0, K <= 18432, group_size a power of two >= 128, rank even <= 256);
 * otherwise GLOWQ_EUNSUPPORTED.
 */
#define GLOWQ_CHAIN_ACC_COPIES 16
#define GLOWQ_CHAIN_ACC_STRIDE 256
#define GLOWQ_CHAIN_ACC_BYTES ((GLOWQ_CHAIN_ACC_COPIES * GLOWQ_CHAIN_ACC_STRIDE + 8) * 8)
#define GLOWQ_CHAIN_PRO_PLAIN 0
#define GLOWQ_CHAIN_PRO_ACC 1
#define GLOWQ_CHAIN_PRO_NORM_ACC 2
#define GLOWQ_CHAIN_EPI_NONE 0
#define GLOWQ_CHAIN_EPI_RESIDUAL 1
#define GLOWQ_CHAIN_EPI_SWIGLU 2
typedef struct glowq_chain_t {
  int prologue, epilogue;
  const void* norm_weight; /* PRO_NORM_ACC: [K] fp16 */
  float eps;
  const void* acc_in;      /* PRO_ACC, PRO_NORM_ACC */
  void* resid;             /* EPI_RESIDUAL: [N] fp16, read and written */
  const void* next_norm_weight; /* EPI_RESIDUAL: [N] fp16 or NULL */
  const void* next_Rt;     /* epilogues: [N, rank] fp16 or NULL (no projection wanted) */
  void* acc_out;           /* with next_Rt */
  void* act;               /* EPI_SWIGLU: [N] fp16 */
} glowq_chain_t;
int glowq_w4a16_group_forward_chained(const void* x, const void* r, const glowq_member_t* members, int n_members, int K,
                                      int group_size, int rank, float alpha, const glowq_chain_t* chain, void* stream);

/* *next_token = index of the first maximum of logits[0..n); then *token = *next_token and *pos += 1 (each if non-NULL). */
int glowq_argmax_advance(const void* logits, int n, int64_t* next_token, int64_t* token, int64_t* pos, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* GLOWQ_W4A16_H_ */
