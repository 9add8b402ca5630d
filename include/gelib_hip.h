/*
 * gelib_hip.h -- C ABI of the MI355X (gfx950) Clebsch-Gordan product library, libgelib_hip.so.
 *
 * This is the drop-in boundary for GElib's device seam: each entry point takes the place of one of
 * the reference's GPU launchers (or of the loop of launches the reference makes at SO3vec level).
 * Plain pointers and sizes only; no C++ or torch types.  All tensors are complex float32, stored
 * interleaved (re,im), viewed as 5-D (batch, grid0, grid1, 2l+1, channels) exactly like the views the
 * reference hands to its launchers (cuda/GPUtensor.hpp:31-38), with strides counted in complex
 * elements and stride 0 meaning "broadcast along this dimension" (core/Gpart.hpp:168-185).
 *
 * Every call is asynchronous on the HIP stream passed in (NULL = the default stream) and returns 0 or
 * one of the gelib_hip_status codes without printing or throwing.  Device memory: the first call for a
 * new coefficient table or a new SO3vec type signature on a device computes its tables and uploads them
 * (one allocation and one synchronous copy, kept for the life of the process); gelib_hip_gather_map_create
 * allocates the map it returns; gelib_hip_malloc allocates what it is asked for; a backward call whose gradient
 * destination broadcasts (see below) takes a temporary that the library keeps per (device, stream).  No other call
 * allocates, frees or synchronises: the channel-mixing entry points take their workspace from the caller.
 *
 * Gradient destinations that broadcast: xg (or yg) with extent 1 along a leading dimension where the other tensors of
 * the call have extent E > 1 is the gradient of an operand shared along that dimension (core/Gpart.hpp:168-185) and
 * receives the SUM over it.  The library forms one gradient per cell with the same kernels as without the broadcast,
 * in a packed temporary of its own (at most "bcast_scratch_kb" KiB, 64 MiB unless set; larger batches are taken in
 * chunks), and adds those up with a two-stage reduction whose order of additions is fixed: same bits every run, no
 * atomics.  The temporary is allocated by the first such call on a (device, stream) pair -- make that call outside
 * stream capture -- grown when a later call needs more, and kept until the process ends; calls on one stream share it
 * in stream order.
 */
#ifndef GELIB_HIP_H
#define GELIB_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct gelib_part_desc {
  void *ptr;          /* device pointer to the first complex element                          */
  int64_t dims[5];    /* (batch, grid0, grid1, 2l+1, channels); a 3-D part has grid0=grid1=1  */
  int64_t strides[5]; /* in complex elements; 0 broadcasts the dimension                      */
} gelib_part_desc;

enum gelib_hip_status {
  GELIB_HIP_OK = 0,
  GELIB_HIP_ERR_NULL = 1,          /* null descriptor or data pointer                                              */
  GELIB_HIP_ERR_ODD_DIM = 2,       /* dims[3] is not 2l+1 (SO3/SO3part.hpp:166-170)                                  */
  GELIB_HIP_ERR_TRIANGLE = 3,      /* |l1-l2| <= l <= l1+l2 not satisfied (cuda/SO3part_addCGproduct.cu:210)         */
  GELIB_HIP_ERR_DIAG_CHANNELS = 4, /* DiagCGproduct with n1 != n2 (SO3/SO3part.hpp:282)                              */
  GELIB_HIP_ERR_CHANNELS = 5,      /* offs + n_out exceeds the product's channels (cuda/SO3part_addCGproduct.cu:214) */
  GELIB_HIP_ERR_BATCH = 6,         /* batch dimensions cannot be reconciled (core/CGproduct.hpp:49)                  */
  GELIB_HIP_ERR_GRID = 7,          /* grid dimensions cannot be reconciled (core/CGproduct.hpp:50)                   */
  GELIB_HIP_ERR_DEVICE = 8,        /* a pointer is not device memory of the current GPU                              */
  GELIB_HIP_ERR_PARTS = 9,         /* too many parts, a repeated l, or l above the supported maximum                 */
  GELIB_HIP_ERR_RUNTIME = 10,      /* a HIP call failed; see gelib_hip_last_runtime_error()                          */
  GELIB_HIP_ERR_BROADCAST_DEST = 11, /* the destination has a dimension of extent > 1 with stride 0 (an expanded view) */
  GELIB_HIP_ERR_ARG = 12,          /* negative offset, negative stride or other malformed argument                   */
  GELIB_HIP_ERR_WORKSPACE = 13,    /* workspace missing, not 16-byte aligned or smaller than the size query says     */
  GELIB_HIP_ERR_TOO_LARGE = 14,    /* sizes beyond the stated maximum of gelib_hip_part_mix_channels_static          */
  GELIB_HIP_ERR_UNSUPPORTED = 15   /* gelib_hip_so3vec_cg_linear_fwd / _bwd: shapes outside what the call takes      */
};

#define GELIB_HIP_MAX_L 32          /* largest l of an operand part                     */
#define GELIB_HIP_MAX_PARTS 33      /* parts per operand SO3vec: every l from 0 to GELIB_HIP_MAX_L   */
#define GELIB_HIP_MAX_OUT_PARTS 65  /* parts of the product / gradient SO3vec: l up to 2 GELIB_HIP_MAX_L */

/* Message for a status code (static storage). */
const char *gelib_hip_strerror(int status);
/* Text of the last HIP runtime error seen by this thread ("" if none). */
const char *gelib_hip_last_runtime_error(void);
/* Library version string. */
const char *gelib_hip_version(void);

/*
 * Host copy of the coefficient matrix <l1 m1; l2 m2 | l m1+m2>, row-major (2l1+1) x (2l2+1) float,
 * zero where |m1+m2| > l.  Same values the kernels use.  Replaces SO3CGbank::get<float>(l1,l2,l,0)
 * (SO3/SO3CGbank.hpp:33-42, 58-95).
 */
int gelib_hip_cg_matrix(int l1, int l2, int l, float *out);

/*
 * Type arithmetic of the product: n_out[l] for l = 0..len-1 (core/Gtype.hpp:115-138).
 * maxl < 0 keeps every l.  Returns the number of parts, or a negative status.
 */
int gelib_hip_so3type_product(int diag, int nx, const int *lx, const int *cx, int ny, const int *ly, const int *cy,
                              int maxl, int64_t *n_out, int len);

/* ---- part level ---------------------------------------------------------------------------------------------
 * accumulate != 0 : reference semantics, add into the destination.
 * accumulate == 0 : overwrite the destination block (channels offs .. offs+n_out-1 of r, or all of xg / yg)
 *                   without reading it, for callers that would otherwise zero-fill first.
 */

/* r[m1+m2, offs+i*n2+j] += C[m1,m2] x[m1,i] y[m2,j].
 * Replaces SO3part_addCGproduct_cu(r,x,y,offs,stream) (cuda/SO3part_addCGproduct.cu:187). */
int gelib_hip_so3part_cg_fwd(const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y, int offs,
                             int accumulate, void *stream);
/* xg[m1,i] += sum_{j,m2} C[m1,m2] g[m1+m2, offs+i*n2+j] conj(y[m2,j]).
 * Replaces SO3part_addCGproduct_back0_cu(xg,g,y,offs,stream) (cuda/SO3part_addCGproduct_back0.cu:224). */
int gelib_hip_so3part_cg_back0(const gelib_part_desc *xg, const gelib_part_desc *g, const gelib_part_desc *y,
                               int offs, int accumulate, void *stream);
/* yg[m2,j] += sum_{i,m1} C[m1,m2] g[m1+m2, offs+i*n2+j] conj(x[m1,i]).
 * Replaces SO3part_addCGproduct_back1_cu(yg,g,x,offs,stream) (cuda/SO3part_addCGproduct_back1.cu:123). */
int gelib_hip_so3part_cg_back1(const gelib_part_desc *yg, const gelib_part_desc *g, const gelib_part_desc *x,
                               int offs, int accumulate, void *stream);

/* r[m1+m2, offs+i] += C[m1,m2] x[m1,i] y[m2,i].  Fills the seam the reference leaves empty
 * (SO3part::add_DiagCGproduct_dev, SO3/SO3part.hpp:324-326); semantics from SO3/SO3part.hpp:276-290. */
int gelib_hip_so3part_diagcg_fwd(const gelib_part_desc *r, const gelib_part_desc *x, const gelib_part_desc *y,
                                 int offs, int accumulate, void *stream);
/* SO3/SO3part.hpp:292-306 (seam SO3/SO3part.hpp:328-330). */
int gelib_hip_so3part_diagcg_back0(const gelib_part_desc *xg, const gelib_part_desc *g, const gelib_part_desc *y,
                                   int offs, int accumulate, void *stream);
/* SO3/SO3part.hpp:308-322 (seam SO3/SO3part.hpp:332-334). */
int gelib_hip_so3part_diagcg_back1(const gelib_part_desc *yg, const gelib_part_desc *g, const gelib_part_desc *x,
                                   int offs, int accumulate, void *stream);

/* ---- SO3vec level: every (l1,l2,l) triple in one call ------------------------------------------------------------
 * Part lists may come in any order; l is read from dims[3].  Triples are enumerated l1 ascending, l2 ascending,
 * l ascending, each writing its block at the running per-l channel offset; a product part that is absent is
 * skipped without moving any other offset (core/Gvec.hpp:311-321).
 */

/* Replaces the loop of Gpart_add_CGproduct calls in Gvec::add_CGproduct (core/Gvec.hpp:311-321). */
int gelib_hip_so3vec_cg_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                            const gelib_part_desc *y, int accumulate, void *stream);
/*
 * Both gradients in one pass over g.  xg (nx parts, shaped like x) and yg (ny parts, shaped like y); either
 * list may be NULL to compute only the other, which then replaces Gvec::add_CGproduct_back0
 * (core/Gvec.hpp:323-333) resp. add_CGproduct_back1 (core/Gvec.hpp:335-345).
 */
int gelib_hip_so3vec_cg_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, int ng, const gelib_part_desc *g,
                            int nx, const gelib_part_desc *x, int ny, const gelib_part_desc *y, int accumulate,
                            void *stream);
/* Gvec::add_DiagCGproduct (core/Gvec.hpp:358-367). */
int gelib_hip_so3vec_diagcg_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                                const gelib_part_desc *y, int accumulate, void *stream);
/* Gvec::add_DiagCGproduct_back0 / _back1 (core/Gvec.hpp:369-389). */
int gelib_hip_so3vec_diagcg_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, int ng,
                                const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny,
                                const gelib_part_desc *y, int accumulate, void *stream);

/* ---- producer of the usual second operand: spherical harmonics ----------------------------------------------------------
 * r[.., l+m, j] += Y_l^m(x[.., :, j] / |x[.., :, j]|), m = -l..l, l read from r's dims[3].  x is float32 viewed 5-D
 * (batch, grid0, grid1, 3, channels) with strides in floats; leading dimensions of extent 1 broadcast.  A vector on
 * the polar axis contributes only m = 0, as in the reference.  accumulate == 0 overwrites r.  The Legendre values
 * are the reference's unnormalised floats, so like the reference the result overflows float32 from l = 30 on.
 * Replaces addSPharm_cu(r, x, stream) (cuda/SPharm.cu:88-123; CPU form SO3/SO3part.hpp:340-403) without its limits of
 * 1024 channels and n(l+1)(l+2)/2 floats of shared memory. */
int gelib_hip_so3part_spharm(const gelib_part_desc *r, const float *x, const int64_t xdims[5],
                             const int64_t xstrides[5], int accumulate, void *stream);

/* ---- consumer of a product: channel mixing ----------------------------------------------------------------------------
 * r[row, o] = sum_c x[row, c] V[c, o], row = 0..rows-1 (the flattened (batch, grid, m) index of a part), overwriting r.
 * adjoint == 0: V = w, a row-major (n_in, n_out) complex matrix: the torch.matmul(part, W) of SO3vec.__mul__ /
 * SO3linear (python/src/gelib/SO3vec.py:174-177, python/src/gelib/SO3weights.py:75-85).  adjoint != 0: w is
 * (n_out, n_in) and V = w^H: the gradient of that matmul with respect to the part (torch's autograd forms it in the
 * reference).  Row strides in complex elements.  n_in must be even and the rows of x 16-byte aligned (else
 * GELIB_HIP_ERR_ARG).  workspace: device memory of at least gelib_hip_part_mix_workspace_bytes(0, rows, n_in, n_out)
 * bytes, 16-byte aligned, that receives the matrix re-packed for the matrix cores; the kernels of the call read it, so
 * it must stay untouched until they have run on `stream` (a buffer from a stream-ordered allocator does).  The library
 * allocates nothing for this call (GELIB_HIP_ERR_WORKSPACE if the buffer is missing or too small). */
int gelib_hip_part_mix_channels(void *r, const void *x, const void *w, int64_t rows, int n_in, int n_out,
                                int64_t r_row_stride, int64_t x_row_stride, int adjoint, void *workspace,
                                uint64_t workspace_bytes, void *stream);
/* gelib_hip_part_mix_channels for callers that cannot allocate device memory and so have no workspace to pass: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels, same results bit for bit; the re-packed matrix goes into an 8 MiB array that
 * is part of the library's device image (each GPU the library runs on holds its own copy until the process ends), so the
 * call allocates nothing -- neither directly nor through any library routine.  Limit: the packed matrix must fit, i.e.
 * gelib_hip_part_mix_workspace_bytes(0, rows, n_in, n_out) <= 8 MiB (16 bytes per pair of channels: n_in * n_out up to
 * 524288 when both are multiples of 16), else GELIB_HIP_ERR_TOO_LARGE.  All calls on one GPU share that GPU's array:
 * calls that may overlap there (two streams, two host threads) race on it and must be ordered by the caller.  The
 * first call on a device asks the runtime for the array's address on that device (no allocation). */
int gelib_hip_part_mix_channels_static(void *r, const void *x, const void *w, int64_t rows, int n_in, int n_out,
                                       int64_t r_row_stride, int64_t x_row_stride, int adjoint, void *stream);
/* wg[c, o] = sum over the rows of conj(x[row, c]) g[row, o], overwriting the row-major (n_in, n_out) matrix wg: the
 * gradient of the same matmul with respect to W (torch's autograd forms it in the reference).  Same conditions on
 * n_in and x.  The rows are summed in ranges whose partial sums are added in a fixed order: the result does not depend
 * on timing.  workspace: at least gelib_hip_part_mix_workspace_bytes(1, rows, n_in, n_out) bytes for those partial sums,
 * same rules as above. */
int gelib_hip_part_mix_channels_wgrad(void *wg, const void *x, const void *g, int64_t rows, int n_in, int n_out,
                                      int64_t x_row_stride, int64_t g_row_stride, void *workspace,
                                      uint64_t workspace_bytes, void *stream);
/* Bytes of workspace the two calls above need: kind 0 for gelib_hip_part_mix_channels (either value of adjoint; n_in and
 * n_out as passed to that call), kind 1 for gelib_hip_part_mix_channels_wgrad.  0 for empty shapes or an unknown kind. */
uint64_t gelib_hip_part_mix_workspace_bytes(int kind, int64_t rows, int n_in, int n_out);

/* ---- CGproduct followed by the weight matrices, in one pass ---------------------------------------------------------------
 * out_l[.., m, o] (+)= sum over c of P_l[.., m, c] w_l[c, o] with P = CGproduct(x, y) restricted to the l of the parts of
 * r, its channels c in the order of core/Gvec.hpp:311-321 -- what the model code of the reference writes as
 * CGproduct(x, y, maxl) * W (python/src/gelib/SO3vec.py:174-177 followed by the per-part matmul of SO3vec.__mul__ with an
 * SO3weights) -- without ever storing P.  r: nr parts (.., 2l+1, n_out_l) that receive the result; w[k] belongs to r[k]:
 * device pointer to the row-major (tau_l, n_out_l) complex matrix, tau_l = channels of part l of the product (host array
 * of nr pointers).  workspace: device memory of at least gelib_hip_so3vec_cg_linear_workspace_bytes(...) bytes, 16-byte
 * aligned, for the matrices re-packed for the matrix cores (same rules as for gelib_hip_part_mix_channels; the library
 * allocates nothing per call).  Taken by the fused kernel: r with every l = 0..4 and at most 16 channels per part,
 * operand parts with l <= 4 and at most 16 channels, contiguous channels, leading dimensions that collapse into one
 * index.  Anything else returns GELIB_HIP_ERR_UNSUPPORTED with nothing launched: the caller then forms the product with
 * gelib_hip_so3vec_cg_fwd and mixes each part with gelib_hip_part_mix_channels.  The sums over c run in a fixed order
 * (ascending c per row, in float32 on the matrix cores); results agree with the two-call form to rounding, not bit for
 * bit. */
int gelib_hip_so3vec_cg_linear_fwd(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x, int ny,
                                   const gelib_part_desc *y, const void *const *w, int accumulate, void *workspace,
                                   uint64_t workspace_bytes, void *stream);
/* Bytes of workspace the call above needs for these parts (256 per product channel plus 4096 per part, and a copy of x
 * rounded up to groups of 32 cells); 0 when the
 * descriptors are malformed or r does not have exactly the parts l = 0..4. */
uint64_t gelib_hip_so3vec_cg_linear_workspace_bytes(int nr, const gelib_part_desc *r, int nx, const gelib_part_desc *x,
                                                    int ny, const gelib_part_desc *y);

/*
 * Backward pass of the call above in bounded memory: with out_l = P_l w_l, P = CGproduct(x, y), and g_l the gradient of
 * out_l (ng parts, n_out_l channels each):
 *     xg, yg (+)= the gradients of x and y          (Gvec::add_CGproduct_back0 / _back1, core/Gvec.hpp:323-345, applied
 *                                                    to gP_l = g_l w_l^H, which torch's autograd forms in the reference),
 *     wg[k]  (+)= sum over the rows of P_l^H g_l     (the gradient of the matmul of python/src/gelib/SO3vec.py:174-177
 *                                                    with respect to the matrix; w[k] and wg[k] belong to g[k]).
 * Any of xg, yg, wg may be NULL.  Neither P nor gP is ever held at full size (25 GB each at the headline type): the
 * batch is taken in chunks whose product fits the workspace -- the forward kernels form a chunk's product there, the
 * matrix-gradient kernel reads it, gP overwrites it in place and the backward kernels read that -- so the call moves the
 * same bytes as the four separate calls and runs at their speed, in the memory of one chunk.  (One kernel that keeps the
 * product on chip throughout would be no faster on this GPU: it needs two matrix products of 12.3 MFLOP per cell and
 * three product-sized contractions on the vector unit, and for float32 the two units do not run at the same time.)
 * workspace: 256-byte aligned device memory; gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(..., batch_chunk) tells the
 * bytes that let the call take batch_chunk batch entries at a time (<= 0: the whole batch at once); with less, the call
 * takes smaller chunks, and GELIB_HIP_ERR_WORKSPACE when not even one batch entry fits.  Conditions
 * (GELIB_HIP_ERR_UNSUPPORTED otherwise, nothing launched): every tensor has the full batch and grid extents, the parts of
 * g are packed along (batch, grid, m) with 16-byte aligned rows, and the channel counts of the product's parts and of
 * g's parts are even.  Operand shapes are not restricted to those of the fused forward kernel.  The sums of wg over the
 * chunks are added in the order of the chunks: results do not depend on timing.
 */
int gelib_hip_so3vec_cg_linear_bwd(const gelib_part_desc *xg, const gelib_part_desc *yg, void *const *wg, int ng,
                                   const gelib_part_desc *g, int nx, const gelib_part_desc *x, int ny,
                                   const gelib_part_desc *y, const void *const *w, int accumulate, void *workspace,
                                   uint64_t workspace_bytes, void *stream);
uint64_t gelib_hip_so3vec_cg_linear_bwd_workspace_bytes(int ng, const gelib_part_desc *g, int nx, const gelib_part_desc *x,
                                                        int ny, const gelib_part_desc *y, int64_t batch_chunk);

/* ---- gather: sums of slices along the batch or a grid dimension ---------------------------------------------------------
 * A gather map is a list of (source, target) pairs with 0 <= source < n_in, 0 <= target < n_out (the arguments of
 * cnine::GatherMapB(sources, targets), python/bindings/gather_map_py.cpp:17-18).  create() checks the indices, sorts the
 * pairs by target (and, for the inverse map, by source), keeping their order within one index, and copies both
 * forms to the current device; the handle is valid on that device until destroy().  Host pointers. */
int gelib_hip_gather_map_create(const int32_t *sources, const int32_t *targets, int64_t npairs, int n_in, int n_out,
                                void **map);
int gelib_hip_gather_map_destroy(void *map);
/*
 * r[.., t, ..] += sum over the pairs (s, t) of x[.., s, ..] along dimension dim of the 5-D views (0 = batch,
 * 1..2 = grid); all other dimensions of r and x agree, dims[dim] is n_out for r and n_in for x.  Replaces
 * Gpart::add_gather(x, gmap, d) with dim = d + 1 (core/Gpart.hpp:556-558).  inverse != 0 runs the map backwards
 * (r has n_in slices, x n_out): Gpart::add_gather_back(g, gmap, d) (core/Gpart.hpp:560-562).  Every output element is
 * summed by one thread in the order of the pairs, so results are reproducible; accumulate == 0 overwrites r,
 * including slices that no pair targets (they become zero).  The loop the reference calls, cnine::GatherSlices, is
 * not in its tree: the semantics here are those of its call sites and of python/docs/source/SO3partArr.rst:97-127
 * with unit weights.
 */
int gelib_hip_part_gather(const gelib_part_desc *r, const gelib_part_desc *x, const void *map, int dim, int inverse,
                          int accumulate, void *stream);

/*
 * Device memory helpers for host code that does not include the HIP headers itself (the C++ mirror of the
 * reference's classes uses them where the reference relies on cnine's device transport, e.g. the
 * TensorView(x, dev) constructor used at SO3/SO3part.hpp:182-183).  kind: 0 host->device, 1 device->host,
 * 2 device->device.  All synchronous.
 */
int gelib_hip_malloc(void **ptr, uint64_t bytes);
int gelib_hip_free(void *ptr);
int gelib_hip_memcpy(void *dst, const void *src, uint64_t bytes, int kind);
int gelib_hip_memset(void *ptr, int value, uint64_t bytes);
int gelib_hip_synchronize(void);

/*
 * Lends the library `bytes` of device memory (256-byte aligned) for its scratch on `stream` of the current device, in
 * place of the buffers it would allocate itself: the per-cell gradients of a destination that broadcasts (first half) and
 * the partial sums of backward launches with few cells (second half).  No counterpart in the reference; it is for callers
 * that record calls into a HIP graph (a recorded call takes no scratch of the library's own, see the top of this file,
 * and falls back to slower routes: with lent memory it runs exactly as an eager call does) and for callers that want
 * every allocation in their own hands.  The memory stays the caller's and must outlive every call and every graph that
 * uses it; a call whose need exceeds its half takes the library's own scratch (eager) or the scratch-free route
 * (recorded).  ptr = NULL or bytes = 0 takes the loan back.  Needs per call: 64 MiB at most for the first half
 * ("bcast_scratch_kb"), 16 x cells x (size of x + size of y per cell) bytes at most for the second (fewer than 1024 cells).
 */
int gelib_hip_set_stream_workspace(void *stream, void *ptr, uint64_t bytes);

/*
 * Tuning / introspection (no counterpart in the reference).
 * gelib_hip_set_option("force_generic", 1) routes every call through the shape-agnostic kernels;
 * "check_pointers" (default 1) switches the device-pointer validation of every call off (0) or on: with 1 an
 * allocation that has passed once is remembered (the last 64 of them), so repeated calls on the same buffers make no
 * driver calls; a buffer that was freed behind the library's back and handed out again smaller at the same address
 * still passes until its entry is pushed out -- gelib_hip_free forgets the entry, setting the option (to any value)
 * forgets all of them, and 2 asks the driver on every call (about 30 us per call instead of 3).
 * "bcast_scratch_kb": KiB the temporary of a broadcast gradient destination may take (0 restores 64 MiB);
 * "bcast_reduce" (1/0): 0 sums such a destination inside the shape-agnostic kernels, one cell after the other.
 * Tuning knobs of the fast families (0 restores the built-in choice unless noted): "unrolled_fwd" / "unrolled_bwd" /
 * "staged_fwd" / "staged_bwd" / "diag6" / "onepair" (1/0: use the family), "fwd_block_bytes", "fwd_lds_bytes", "fwd_tile",
 * "fwd_cell_tile" (cells per tile of the unrolled forward launch, 0 = one tile, -1 = chosen by the channel counts, the
 * default), "bwd_lds_target" (LDS bytes per block the unrolled backward kernels aim at when they choose their cells per
 * block), "bwd_min_runs" (runs of 64 lane slots such a block should have at least, 0 = no such rule), "unrolled_bwd_l6" / "unrolled_fwd_l6" (1/0: the backward / forward kernel for operands up to l = 6),
 * "staged_fwd_tile" (1, 2, 4), "staged_fwd_threads", "staged_fwd_coeffs_lds" (1/0), "staged_fwd_lds_target",
 * "staged_bwd_lds_target", "staged_bwd_threads" (256, 512, 1024), "staged_bwd_stripes" (0 never, otherwise wherever they
 * apply), "staged_bwd_atomic" (1/0: allow the single-pass backward kernels that add with LDS float atomics; off by
 * default, so that results do not depend on timing), "staged_bwd_pairs" (1/0: the pair-wise one of those),
 * "pairwise_bwd" (one launch of the single-pair kernels per pair of parts, backward and -- for operand l above 7 --
 * forward: 0 never, 1 for operand l above 7, 2 backward wherever every pair qualifies), "onepair_mfma" (1/0: the
 * matrix-core form of the single-pair kernel, built for 4 x 4, 8 x 2, 8 x 8, 4 x 16, 8 x 16, 16 x 8 and 16 x 16 channels), "onepair_mfma_fwd" (1/0:
 * its forward kernel), "onepair_mfma_paired" (1/0: row numbers taken in pairs when l1 = l2), "unrolled_bwd_one" (1/0: the
 * backward kernel built for calls with one triple), "diag6_sets" (1/0: the Diag backward kernel with compile-time sets of
 * l2 per wave), "diag6_l8" (0: Diag products above l = 6 are always split at l = 6; 1: operands up to l = 4 run forward in
 * one launch of the kernels built for products up to l = 8; 2: backward too), "diag6_hi" (1/0: the part l = 7..12 of a
 * split Diag product runs on the lane-per-channel kernels built for it), "diag6_small" (1/0: Diag kernels that give a wave, not a
 * block, a cell and channel group: operands up to l = 2, backward up to l = 4), "diag6_one_channel" (1/0: a CGproduct in which every part of exactly one operand has one
 * channel runs on the lane-per-channel Diag kernels), "unrolled_bwd_one_wide" (1/0: the wave-per-cell backward kernel
 * for calls with one triple and 16 or 32 channels in the second operand) and "unrolled_bwd_one_wide_cells" (cells from
 * which it is used, 4096), "unrolled_bwd_split" (1/0: launches with few cells deal a cell's pairs to several blocks),
 * "unrolled_bwd_split_below" (blocks below which they do, 1024) and "unrolled_bwd_split_max" (blocks per cell at most,
 * 16), "unrolled_bwd_l6_split" (1/0: a product above l = 6 of operands above l = 4 goes backward in two launches of the
 * unrolled kernels, l <= 6 and l = 7..12), "fwd_narrow_decline" (1/0: products with
 * at most four channel pairs per block go forward on the any-l kernels).  Unknown names return
 * GELIB_HIP_ERR_ARG.  Options are process-wide.
 * gelib_hip_last_path() tells which kernel family the last call of this thread used
 * (0 = none, 1 = generic, 2 = unrolled small-l kernels, 3 = staged any-l kernels, 4 = lane-per-channel Diag
 * kernels for operand l up to 6, 5 = single-pair kernels for large l, 6 = the product fused with the weight matrices).
 */
int gelib_hip_set_option(const char *name, int value);
int gelib_hip_last_path(void);

#ifdef __cplusplus
}
#endif
#endif
