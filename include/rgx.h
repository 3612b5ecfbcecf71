/*
 * rgx.h -- C ABI of librgx.so: the MI355X (gfx950) implementation of the
 * RayGaussX differentiable Gaussian ray-marching renderer.
 *
 * Every entry point replaces a piece of the reference's OptiX/CuPy host glue
 * (paths relative to the reference tree).  Conventions:
 *   - all pointers are DEVICE pointers unless the parameter is documented as
 *     "host"; every entry point that launches work makes the device that owns
 *     its first device pointer current for the duration of the call (and
 *     restores the caller's), so a binding need not call hipSetDevice itself;
 *   - `stream` is a hipStream_t passed as void* (0 = the null stream); every
 *     call only enqueues work on it and never synchronises, except the two
 *     explicitly synchronous read-back helpers;
 *   - the caller owns every buffer, including the workspaces whose sizes the
 *     *_bytes queries return; the library never allocates device memory;
 *   - return 0 on success or a negative RGX_E* code; nothing throws or exits.
 *     rgx_strerror() names a code, rgx_last_hip_error() returns the hipError_t
 *     behind the calling thread's last RGX_EHIP.
 * Calls are thread-compatible (the autograd engine calls the backward from
 * its own thread); two calls that share a workspace must be ordered by the
 * stream.
 */
#ifndef RGX_H
#define RGX_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RGX_ABI_VERSION 6

#define RGX_OK 0
#define RGX_EINVAL -1     /* bad argument (null pointer, negative size, unsupported degree ...) */
#define RGX_EWORKSPACE -2 /* workspace too small or misaligned */
#define RGX_EHIP -3       /* a HIP runtime call failed; see rgx_last_hip_error() */
#define RGX_ELIMIT -4     /* a size beyond the fixed limits of rgx_march_backward_noalloc() */

/* Launch constants of one view.  Mirrors the camera part of `Params`
 * (optix_raycasting/cuda_train/forward/gaussians_aabb.h:14-44) as filled at
 * optix_raycasting/optix_utils.py:252-266.  Host struct. */
typedef struct RgxCamera {
    float eye[3];       /* camera.camera_center */
    float u[3];         /* world_view_transform[:3,0]  (camera right, world space) */
    float v[3];         /* world_view_transform[:3,1]  (camera down) */
    float w[3];         /* world_view_transform[:3,2]  (camera forward) */
    float tan_half_fov_x, tan_half_fov_y, principal_x, principal_y; /* cam_intr */
    int32_t width, height; /* already multiplied by the supersampling factors */
} RgxCamera;

/* Marching constants.  dt_step / dynamic_sampling / max_prim_slice /
 * white_background are `Params` fields; t_eps is TRANSMITTANCE_EPSILON
 * (gaussians_aabb.h:4, 0.001f in the reference) made a run-time value. Host struct. */
typedef struct RgxMarch {
    float dt_step;
    int32_t dynamic_sampling;
    int32_t max_prim_slice;
    int32_t white_background;
    float t_eps;
    int32_t record_format; /* of the sample sums a forward leaves in its record for the backward (not in the
                              reference, which keeps no record): 0 float colour sums, 32 KiB per slab iteration of a
                              tile; 1 half-precision colour sums with a power-of-two scale per ray and 16 samples,
                              20.5 KiB.  The forward and the backward of a view must be given the same value. */
} RgxMarch;

/* Optional device-side counters, accumulated (not reset) by the march kernels. */
typedef struct RgxStats {
    unsigned long long hit_pairs;     /* sum over blended slabs of the hit-list length (a forward without a record
                                         collects a crowded slab half by half and never collects, or counts, the
                                         second half for a ray that ends in the first: a few per cent fewer in
                                         dense scenes; with a record every list is whole, as in the reference) */
    unsigned long long slabs;         /* slabs blended */
    unsigned long long empty_slabs;   /* collect queries that found nothing */
    unsigned long long overflow_rays; /* collect queries truncated at max_prim_slice */
    unsigned long long rays_hit;      /* rays whose first-hit query found a Gaussian */
    unsigned long long nodes_visited; /* BVH nodes fetched by all queries */
    unsigned long long candidates;     /* Gaussians gathered per tile and slab iteration (filter passes) */
    unsigned long long candidates_hit; /* ... of which at least one ray of the tile hit */
    unsigned long long replay_lost;    /* tiles whose backward did not consume its hit-list record exactly (expect 0) */
    unsigned long long grad_atomics;   /* fp32 atomic adds of the backward's gradient scatter to memory (14 per Gaussian and
                                          window when it replays a record; 14 per Gaussian, slab and 4x4 pixel row otherwise) */
} RgxStats;

int rgx_abi_version(void);
const char *rgx_strerror(int code);
int rgx_last_hip_error(void);

/* ---- per-Gaussian kernels ------------------------------------------------ */

/* Replaces ellipsoids_bbox_from_quat (optix_utils.py:36-109): k-sigma AABB of
 * every Gaussian plus the scene bounding box.  bboxes (N,6) = xmin,ymin,zmin,
 * xmax,ymax,zmax; bb_min/bb_max (3) device floats.  Any output may be NULL. */
int rgx_aabb(const float *pos, const float *scale, const float *quat, const float *dens, int64_t n,
             float sigma_threshold, float *bboxes, float *bb_min, float *bb_max, void *stream);

/* Replaces forward_sh (utils/sh_utils.cu:122-216) as launched by compute_cupy_rgb
 * (render_optix.py:19-32).  sh is (N,3,K) channel-major, K=(degree+1)^2, degree 0..3;
 * sg (N,3,G), sharp (N,G), axis (N,G,3) may be NULL when G == 0.  eye: host float[3]. */
int rgx_sh_forward(const float *eye, const float *pos, const float *sh, const float *sg,
                   const float *sharp, const float *axis, int32_t g, int32_t degree, int64_t n,
                   float *rgb, void *stream);

/* Replaces backward_sh (utils/sh_utils.cu:218-412) as launched by compute_cupy_sh_grad
 * (render_optix.py:34-52).  Writes (does not accumulate) dsh (N,3,K), dpos (N,3) and,
 * when G > 0, dsg / dsharp / daxis.  Keeps the reference's d/dy term of basis 9
 * (sh_utils.cu:367).  eye: host float[3]. */
int rgx_sh_backward(const float *eye, const float *pos, const float *sh, const float *sg,
                    const float *sharp, const float *axis, int32_t g, int32_t degree, int64_t n,
                    const float *drgb, float *dsh, float *dpos, float *dsg, float *dsharp,
                    float *daxis, void *stream);

/* ---- acceleration structure ---------------------------------------------- */

/* Replaces create_acceleration_structure (optix_utils.py:139-142; the OptiX
 * GAS build) together with the AABB pass that feeds it: k-sigma AABBs, scene
 * bbox, 63-bit Morton codes of the centres, radix sort, Karras radix tree,
 * bottom-up refit, skip links.  The result lives in `ws` (device memory of at
 * least rgx_build_workspace_bytes(n) bytes, 256-byte aligned) and stays valid
 * until the next build into the same buffer; reuse it across views. */
int rgx_build_workspace_bytes(int64_t n, size_t *bytes);
int rgx_build(const float *pos, const float *scale, const float *quat, const float *dens, int64_t n,
              float sigma_threshold, void *ws, size_t ws_bytes, void *stream);

/* Same tree over caller-supplied boxes (N,6), the literal signature of
 * create_acceleration_structure(ctx, bboxes) (optix_utils.py:139-142). */
int rgx_build_aabbs(const float *bboxes, int64_t n, void *ws, size_t ws_bytes, void *stream);

/* Replaces update_acceleration_structure(gas, bboxes) (optix_utils.py:144-146; OptiX's
 * accel update): new boxes for the same Gaussians into a workspace that rgx_build / rgx_build_aabbs
 * built for this n.  The tree keeps its shape (sorted order, children); leaf and internal boxes and
 * the scene box are recomputed.  About a third of a build's time; queries stay exact however far the
 * Gaussians moved, the tree only culls worse the further they did.
 * Precondition: `ws` holds a finished tree over exactly n boxes and `bboxes` has n rows.  The first
 * is checked on the device, in stream order, by the refit's first kernel: when it does not hold
 * (workspace never built, built for another n, or left unfinished) no kernel of the refit touches
 * the tree, the workspace is left marked not built -- rgx_scene_bbox then returns RGX_EWORKSPACE --
 * and this call still returns RGX_OK, because the host does not wait for the check. */
int rgx_refit_aabbs(const float *bboxes, int64_t n, void *ws, size_t ws_bytes, void *stream);

/* Synchronous read-back of the scene bbox held in a built workspace
 * (host out[6] = min xyz, max xyz); what bb_min.get()/bb_max.get() returned at
 * optix_utils.py:254-255.  Waits for `stream`.  RGX_EWORKSPACE when the workspace holds no
 * finished tree (never built, or a refit that was refused). */
int rgx_scene_bbox(const void *ws, float *host_out6, void *stream);
/* The build's permutation: order[j] = input index of the j-th Gaussian in Morton order. */
int rgx_build_order(const void *ws, int64_t n, int32_t *order_out, void *stream);
/* Test hook: where a built workspace keeps the tree, as byte offsets from `ws` (host out[6]):
 * 0 boxes (n,6) floats in input order; 1 order (n) uint32; 2 nodes (2n-1) records of 32 bytes
 * {lo[3], left | ~sorted leaf index, hi[3], skip}, internal nodes first, leaf j of the Morton
 * order at n-1+j; 3 parent (2n-1) int32; 4 right child (n-1) int32; 5 the 64-byte header
 * {bb_min[3], bb_max[3], ...}.  Lets a test read a tree back and check it on the host (child
 * boxes inside their parent, skip links, permutation); OptiX's GAS is opaque, so the reference
 * has no counterpart. */
int rgx_build_layout(int64_t n, size_t *host_out6);

/* Replaces the prim packing at optix_utils.py:268-304: the 64-byte PrimData record
 * (gaussians_aabb.h:7-12) of every Gaussian, written in the build's Morton order
 * when `ws` is a built workspace, or in input order when ws == NULL.
 * eye: host float[3].  prims: (N,16) floats, 64-byte aligned. */
int rgx_pack_prims(const void *ws, const float *eye, const float *pos, const float *scale,
                   const float *quat, const float *dens, const float *rgb, int64_t n,
                   float sigma_threshold, float *prims, void *stream);

/* ---- ray march ------------------------------------------------------------ */

/* Scratch for one march launch: the backward's Morton-ordered gradient block (64 bytes per
 * Gaussian) and, sized from n_rays, the order in which the replaying backward takes the image's
 * tiles (largest hit-list record first).  A workspace that only has room for the gradient block
 * (64 n bytes rounded up to 256) is accepted: the tiles then run in launch order.  (The
 * reference's per-ray hit scratch hit_prim_idx, optix_utils.py:306, has no counterpart.) */
int rgx_march_workspace_bytes(int64_t n, int64_t n_rays, int32_t max_prim_slice, size_t *bytes);

/* Optional record of one forward launch, tile_words 32-bit words per 8x8 pixel tile on average
 * (>= 1024, multiple of 4).  Up to 16384 words per tile hold the hit lists: per slab iteration,
 * which Gaussians each 4x4 pixel row hits and each ray's hit bits (16384 is ample for the benchmark
 * scenes).  A backward given the record of its forward replays those lists instead of searching the
 * tree again; tiles whose region overflowed, or whose region was not written by a forward launch
 * with the same number of Gaussians, image size and step, are recomputed.  The role the
 * reference's hit_prim_idx buffer plays between its collect and blend steps (optix_utils.py:306),
 * at a few hundred bytes per tile and slab instead of max_prim_slice ints per ray.
 * What tile_words gives beyond 16384 (at least 8192 more) becomes one pool of 32 KiB slots shared
 * by all tiles: per slab iteration that blends something, the per-sample density and colour sums
 * of its 64 rays.  The backward then reads these back instead of walking the hit lists once more
 * to rebuild them (about a fifth faster; 16384 + 64 * 8192 words per tile hold the benchmark
 * scenes).  Tiles that found the pool empty are replayed from their hit lists alone. */
int rgx_march_records_bytes(int32_t width, int32_t height, int32_t tile_words, size_t *bytes);

/* Replaces launch_pipeline_forward / launch_pipeline_test (optix_utils.py:222-322,
 * 503-601) and the OptiX programs of cuda_train/forward/gaussians_aabb.cu:
 * ray_colors (W*H,3), row-major pixels.  cam, march: host structs.
 * prims: from rgx_pack_prims with the same ws.  records (16-byte aligned, may be NULL):
 * where to write the hit-list record.  stats may be NULL, and should be outside diagnostics:
 * a launch without a statistics block runs kernels that carry no counters (5 % faster). */
int rgx_march_forward(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims,
                      int64_t n, float *ray_colors, void *march_ws, size_t march_ws_bytes,
                      void *records, size_t records_bytes, RgxStats *stats, void *stream);

/* Test hook: rgx_march_forward through the counting kernels, with the counters also kept per ray:
 * ray_counts (W*H, 2) = slabs blended and the sum of their hit-list lengths (the per-ray share of
 * RgxStats.slabs / hit_pairs).  Lets a test tell which rays marched the same slab sequence as a CPU
 * evaluation when the adaptive step makes that depend on the last bit of cbrt / exp. */
int rgx_march_forward_counts(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims,
                             int64_t n, float *ray_colors, void *march_ws, size_t march_ws_bytes, void *records,
                             size_t records_bytes, RgxStats *stats, uint32_t *ray_counts, void *stream);

/* Replaces launch_pipeline_backward + reduce_temp_grads (optix_utils.py:325-500) and
 * cuda_train/backward/gaussians_aabb.cu: gradients of sum(dloss * ray_colors) with
 * respect to density (N), rgb (N,3), position (N,3), scale (N,3), quaternion (N,4),
 * in INPUT order, overwritten.  ray_colors is the forward's output.  records: the record
 * written by the forward launch with the same ws, cam, march and prims, or NULL. */
int rgx_march_backward(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims,
                       int64_t n, const float *ray_colors, const float *dloss, float *ddens,
                       float *drgb, float *dpos, float *dscale, float *dquat, void *march_ws,
                       size_t march_ws_bytes, const void *records, size_t records_bytes,
                       RgxStats *stats, void *stream);

/* rgx_march_backward for callers that cannot allocate device memory or bring a workspace: code
 * under HIP graph capture, tight serving / fine-tuning loops, harnesses that forbid hipMalloc.
 * It has no counterpart in the reference.  Same arguments and results as rgx_march_backward
 * without march_ws: the gradient block and the tile order live in a file-scope device array of
 * the library instead (RGX_NOALLOC_SCRATCH_BYTES, about 64.3 MiB, held by every GPU the library
 * runs on until the process ends).  Limits: n <= RGX_NOALLOC_MAX_GAUSSIANS and width * height <=
 * RGX_NOALLOC_MAX_RAYS, else RGX_ELIMIT.  The call allocates nothing, frees nothing and does not
 * synchronise; it clears the part of the array it uses with a kernel.  All calls on one GPU share
 * that GPU's array: calls that overlap on one GPU (two streams, two threads) race -- order them. */
#define RGX_NOALLOC_MAX_GAUSSIANS (1 << 20)
#define RGX_NOALLOC_MAX_RAYS (1 << 22)
#define RGX_NOALLOC_SCRATCH_BYTES 67444992 /* 64 bytes per Gaussian + 256 + 4 bytes per 8x8 tile * 5/4 + 8192 */
int rgx_march_backward_noalloc(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims,
                               int64_t n, const float *ray_colors, const float *dloss, float *ddens,
                               float *drgb, float *dpos, float *dscale, float *dquat, const void *records,
                               size_t records_bytes, RgxStats *stats, void *stream);

/* Launch faults that do not stop a launch, counted in the march workspace (always, with or without a
 * statistics block) and read back here; synchronous, waits for `stream`.  host_out[0]: tiles whose
 * replaying backward did not consume its hit-list record exactly (the gradient of such a tile is
 * that of the iterations replayed so far); host_out[1]: sweeps of the tree that had to drop nodes
 * because the node stack was full (cannot happen for trees of at most 2^30 leaves; counted so that
 * it would be seen).  rgx_march_forward and rgx_march_viewer clear both at their start;
 * rgx_march_backward clears host_out[0] at its start and adds to host_out[1], which therefore covers
 * the forward and the backward launches since.  A backward into a workspace that no forward has used
 * finds host_out[1] as the memory was: zero a fresh workspace's 256 bytes at offset
 * align256(max(n, 1) * 64) first (the Python mirror allocates its workspaces zeroed).  A workspace with
 * room for the gradient block only keeps no counts (zeros); the array of rgx_march_backward_noalloc
 * cannot be read back. */
int rgx_march_faults(const void *march_ws, size_t march_ws_bytes, int64_t n, uint64_t *host_out2, void *stream);

/* The interactive viewer's two kernels (its GL window and interop stay with the caller).
 * rgx_sh_viewer replaces gui_sh (utils/sh_utils.cu:25-119): rgx_sh_forward on tensors that keep
 * room for max_num_sh coefficients per channel and max_sg_display lobes per Gaussian, of which the
 * first (degree+1)^2 and g are evaluated.
 * rgx_march_viewer replaces the viewer's launch of cuda_gui/gaussians_aabb.cu: the forward march on
 * a black background; frame (W*H uchar4: r, g, b quantised as min(uint(x*256), 255), alpha 255),
 * depth (W*H): sum over the samples of T (1 - w) t (cuda_gui/gaussians_aabb.cu:189-202).
 * march->white_background is ignored. */
int rgx_sh_viewer(const float *eye, const float *pos, const float *sh, const float *sg, const float *sharp,
                  const float *axis, int32_t g, int32_t degree, int32_t max_num_sh, int32_t max_sg_display,
                  int64_t n, float *rgb, void *stream);
int rgx_march_viewer(const void *ws, const RgxCamera *cam, const RgxMarch *march, const float *prims, int64_t n,
                     uint8_t *frame, float *depth, void *march_ws, size_t march_ws_bytes, RgxStats *stats, void *stream);

/* Replaces the per-tensor `tensor[reordering_index]` gathers of PointCloud.reorder_zordercurve and
 * OptimizerManager._reorder_tensors (classes/point_cloud.py:1031-1044, classes/optimizer.py:54-66)
 * by one launch: for each of `count` tensors, dst[i] row j = src[i] row order[j].  src, dst,
 * row_bytes: HOST arrays of `count` device pointers / row sizes in bytes (multiples of 4); all
 * tensors have n rows; dst[i] != src[i].  order: device int64, a permutation of 0..n-1. */
int rgx_gather_rows(int32_t count, const void *const *src, void *const *dst, const int64_t *row_bytes,
                    const int64_t *order, int64_t n, void *stream);

/* Replaces distCUDA2 of the simple-knn extension (submodules/simple-knn/simple_knn.cu:186-222,
 * called at classes/point_cloud.py:252 to initialise the scales): mean_dist2[i] = mean of the
 * squared distances from point i to its three nearest other points (FLT_MAX stands in for a
 * missing neighbour when n < 4, as there).  pos (n,3).  ws from rgx_knn_workspace_bytes. */
int rgx_knn_workspace_bytes(int64_t n, size_t *bytes);
int rgx_dist2_knn3(const float *pos, int64_t n, float *mean_dist2, void *ws, size_t ws_bytes, void *stream);

/* Replaces reduce_supersampling (utils/general_utils.py:489-502) and the clip / 8-bit
 * quantisation that follow it in the inference loop (scripts/test.py:197-200,
 * utils/general_utils.py:167): ray_colors ((width*factor_x)*(height*factor_y), 3) as the march
 * wrote it -> out (height*width, 3), the mean over each pixel's factor_x x factor_y rays, summed in
 * the reference's order; clipped to [0,1] when clip != 0; out8 = uint8(255 * clipped value).
 * Either of out, out8 may be NULL. */
int rgx_reduce_supersampling(const float *ray_colors, int32_t width, int32_t height, int32_t factor_x,
                             int32_t factor_y, int32_t clip, float *out, uint8_t *out8, void *stream);

/* Test hooks: the two OptiX ray queries on caller-supplied segments (origin = eye,
 * host float[3]; dirs (n,3); tlo/thi (n)).  first-hit: optixTrace SBT offset 0
 * (gaussians_aabb.cu:234-247, 370-380), out_t = smallest hit t or -1.  collect:
 * optixTrace SBT offset 1 + __anyhit__ah (gaussians_aabb.cu:282-295, 349-367),
 * counts[i] = number of hits (negated when truncated at cap), ids (n,cap) = INPUT
 * indices in traversal order. */
int rgx_first_hit(const void *ws, const float *prims, int64_t n_prims, const float *eye, int64_t n,
                  const float *dirs, const float *tlo, const float *thi, float *out_t, void *stream);
int rgx_trace_segments(const void *ws, const float *prims, int64_t n_prims, const float *eye, int64_t n,
                       const float *dirs, const float *tlo, const float *thi, int32_t cap,
                       int32_t *counts, int32_t *ids, void *stream);

/* The collect query as the march kernels run it: one 8x8 pixel tile per wavefront, the
 * tile's Gaussians gathered once and tested per ray.  tlo/thi (W*H) give each pixel's
 * segment (thi < tlo: pixel idle); counts (W*H) and ids (W*H,cap) as rgx_trace_segments.
 * uncounted != 0 runs the filter as the kernels launched without a statistics block compile it
 * (with its early exit for entries that no ray's line meets); 0: as the counting kernels do. */
int rgx_collect_tiles(const void *ws, const RgxCamera *cam, const float *prims, int64_t n_prims,
                      const float *tlo, const float *thi, int32_t cap, int32_t *counts, int32_t *ids,
                      int32_t uncounted, void *stream);

/* Test hook for the arithmetic of the hit predicate.  Where a Gaussian's scales and distance are of
 * ordinary size the kernels form the predicate's two quotients and its square root
 * (gaussians_aabb.cu:59-75) with the compiler's own instruction sequences for `/` and sqrtf()
 * minus their handling of extreme exponents.  This counts, over n pairs (a[i], b[i]) of device
 * floats, those for which a / b, 1 / b, sqrt(|a|) or sqrt(2^-40 |a|) so formed differ in any bit
 * from the full sequences; *bad (device, cleared by the caller) receives the count, 0 for operands in range
 * (2^-46 <= |a|, |b| <= 2^46). */
int rgx_check_plain_arith(const float *a, const float *b, int64_t n, uint32_t *bad, void *stream);

/* Measurement hook (no counterpart in the reference): a kernel that issues one VALU instruction over
 * and over on independent registers, for the rate at which this card issues that class of instruction
 * -- the ceiling the march kernels, which are bound by instruction issue, are priced against.
 * kind: 0 v_fma_f32, 1 v_add_f32, 2 v_mov_b32, 3 v_and_b32, 4 v_cmp_lt_f32, 5 v_cndmask_b32,
 * 6 v_max_f32, 7 v_add_f32 with a DPP operand, 8 v_lshlrev_b32, 9 v_exp_f32 (these let the compiler
 * place the operands: a repeated multiplicand and addend, the cheapest case); 10..13 name their
 * registers, because the cost depends on which of the register file's two banks (even and odd
 * numbers) the sources sit in and on whether the previous instruction read the same ones: 10
 * v_fma_f32 acc = x * k + acc with a fresh x from the other bank, 11 v_fma_f32 with three fresh
 * sources from both banks, 12 the same from one bank, 13 v_mul_f32 of two fresh sources (160
 * registers: at most three wavefronts per SIMD).  Launches `waves`
 * wavefronts (rounded up to whole workgroups of four) that each issue iters * 64 of them;
 * *instructions (host) receives the number of wave instructions the launch issues in its loops.
 * `sink` (device, at least one float) keeps the registers live; nothing is written to it for finite
 * inputs.  The caller times the launch with events on `stream`. */
int rgx_probe_valu_rate(int32_t waves, int32_t iters, int32_t kind, float *sink, uint64_t *instructions, void *stream);

/* ---- Morton reordering of the point cloud --------------------------------- */

/* Replaces quantify_pos_min_max + morton_code + argsort (utils/reordering_utils.py:55-104,
 * classes/point_cloud.py:1017-1024): 10 bits per axis on the positions' own min/max,
 * x -> bit 3i, y -> 3i+1, z -> 3i+2; order = stable ascending sort of the codes.
 * codes (N) int64 and order (N) int64 outputs; either may be NULL. */
int rgx_morton_workspace_bytes(int64_t n, size_t *bytes);
int rgx_morton_order(const float *pos, int64_t n, int64_t *codes, int64_t *order, void *ws,
                     size_t ws_bytes, void *stream);

/* ---- measurement ----------------------------------------------------------- */

/* Per-kernel timing with HIP events recorded on the launch stream around the kernels
 * of each entry point (what the reference's commented-out CUDA-event code at
 * optix_utils.py:466-485 and scripts/test.py:109-126 measured).  Off by default.
 * ids: 0 build, 1 sh_forward, 2 pack_prims, 3 march_forward (the k_march_fwd launch
 * only), 4 march_backward (the k_march_bwd launch only), 5 unpermute_grads,
 * 6 sh_backward.  rgx_timing_read waits for the recorded events and returns the
 * summed milliseconds and the number of launches since the last reset. */
int rgx_timing_enable(int on);
int rgx_timing_reset(void);
const char *rgx_timing_name(int id);
int rgx_timing_read(int id, double *total_ms, int64_t *launches);

#ifdef __cplusplus
}
#endif
#endif /* RGX_H */
