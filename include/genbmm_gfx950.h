/*
 * genbmm_gfx950.h — C ABI of libgenbmm_gfx950.so
 *
 * Generalized-semiring batched matrix multiply (log / max / sample / prod-max)
 * and banded-matrix multiply for AMD MI355X (gfx950, CDNA4), as hand-written
 * HIP kernels behind plain C entry points.
 *
 * This library replaces the private pybind11 module `_genbmm` of
 * harvardnlp/genbmm (reference matmul_cuda.cpp:165-172) whose six functions
 * `forward, backward, backbackward, forward_band, backward_band,
 * backbackward_band` return freshly allocated torch tensors.  Here the entry
 * points take raw device pointers instead:
 *
 *   - every pointer is a DEVICE pointer to a dense row-major fp32 (or int32)
 *     buffer that the CALLER allocated; outputs are fully overwritten, they
 *     need no initialisation;
 *   - the library never allocates, frees or synchronises; every call only
 *     enqueues kernels on `stream` (a hipStream_t passed as void*; NULL is the
 *     legacy default stream);
 *   - return value: 0 = enqueued; < 0 = argument error (GENBMM_E_*);
 *     > 0 = the hipError_t reported by the launch;
 *   - calls are re-entrant and thread safe: a pointer declared const is only
 *     read, and the library keeps no mutable global state - except in
 *     genbmm_logbmm_fwd_static, whose fixed workspace is shared by all calls on
 *     a GPU (see there).
 *
 * Dense operands: a is (B, M, K), b is (B, K, N), results are (B, M, N).
 * Banded operands: band data is (B, n, W) with W = lu + ld + 1 and
 * data[b, c, k] = Dense[b, c + k - lu, c]  (reference genbmm/sparse.py:12-30).
 */
#ifndef GENBMM_GFX950_H
#define GENBMM_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Argument errors (negative return values). */
#define GENBMM_OK 0
#define GENBMM_E_NULLPTR (-1) /* a required pointer is NULL            */
#define GENBMM_E_SHAPE (-2)   /* a dimension is < 0 or overflows int32 */
#define GENBMM_E_MODE (-3)    /* unknown semiring mode or kernel path  */
#define GENBMM_E_BAND (-4)    /* negative band width                   */
#define GENBMM_E_TOOBIG (-5)  /* beyond a fixed-size workspace's limit */

/* Banded semiring modes (reference banded_cuda_kernel.cu:42,64,76). */
#define GENBMM_BAND_LOG 0
#define GENBMM_BAND_MAX 1
#define GENBMM_BAND_SAMPLE 2  /* backward only: a drawn index scatters like an arg-max */
#define GENBMM_BAND_MUL 3

/* Library version string, e.g. "genbmm-gfx950 0.1". */
const char* genbmm_version(void);

/* Human-readable text for a return value of any function below. */
const char* genbmm_error_string(int code);

/* ------------------------------------------------------------------ dense */

/*
 * out[b,m,n] = log sum_k exp(a[b,m,k] + b[b,k,n]).
 * Replaces _genbmm.forward(a, b, 0): matmul_cuda.cpp:69-77 ->
 * matmul_cuda_forward mode 0 (matmul_cuda_kernel.cu:465-497, kernel :13-45).
 * The running maximum starts at -1e9 as in the reference (kernel :31), so an
 * output whose terms are all <= -1e9 is -inf.
 *
 * `stats` is an optional fp32 buffer of genbmm_logbmm_stats_size(B,M,K,N)
 * elements.  NULL: the online (running-max) log-sum-exp kernel runs.
 * Non-NULL: its first B*(M+N) elements receive, per batch item, max_k a[m,k]
 * for every m followed by max_k b[k,n] for every n, and the forward uses them
 * to factor exp(a+b) = exp(a-max)*exp(b-max) wherever that is exact to fp32;
 * behind them sit per-tile flags naming the tiles where it is not, which a
 * fix-up launch recomputes with the online kernel's routine, a header naming
 * the kernels that filled the buffer, and - for shapes that run on the matrix
 * cores (M and N at least 96, K at least 16) and do not fit one 128 x 128 tile
 * per batch item - exp(a-max), exp(b-max) and 1/sum, which the backward then
 * reads instead of taking any exponential itself.  Items of one tile (every
 * extent between 64 and 128) keep the maxima alone: forward and backward each
 * form what they need in one launch, and a tile that cannot be factored is
 * redone by the exact routine inside that launch.
 * The contents belong to the library; the buffer takes the place of
 * the reference's (B, M, N) `maxes` output; pass the same buffer, unchanged,
 * to genbmm_logbmm_bwd.
 */
int genbmm_logbmm_fwd(const float* a, const float* b, float* out, float* stats,
                      int B, int M, int K, int N, void* stream);

/*
 * grad_a[b,m,k] = sum_n exp(a[m,k] + b[k,n] - out[m,n]) * g[m,n]
 * grad_b[b,k,n] = sum_m exp(a[m,k] + b[k,n] - out[m,n]) * g[m,n]
 * Replaces the two _genbmm.backward(..., 0) calls plus six transposes of
 * LogMatMul.backward (genmul.py:35-41; matmul_cuda.cpp:79-92;
 * matmul_cuda_kernel.cu:625-664, kernel :159-184).
 * grad_a or grad_b may be NULL (that gradient is then not computed), not both.
 * `stats`: NULL, or the buffer genbmm_logbmm_fwd filled for the same (a, b).
 * It is only read: any number of backward calls, on any streams, may share it.
 * Its header tells which forward kernels filled it; a backward kernel that
 * needs by-products the buffer does not hold (or meets a tile the forward
 * flagged) leaves that tile to the exact routine, so a mismatch costs time,
 * never correctness.  With both gradients requested a matrix-core problem is
 * one launch.
 */
int genbmm_logbmm_bwd(const float* a, const float* b, const float* out,
                      const float* g, const float* stats,
                      float* grad_a, float* grad_b,
                      int B, int M, int K, int N, void* stream);

/* Number of fp32 elements genbmm_logbmm_fwd / _bwd need in `stats`. */
size_t genbmm_logbmm_stats_size(int B, int M, int K, int N);

/*
 * Number of fp32 elements genbmm_samplebmm_fwd needs in its `stats` (never less
 * than genbmm_logbmm_stats_size: the sampling sweep always wants the factors
 * where a forward can leave them, and on a problem whose forward cuts its
 * reduction into pieces - genbmm_logbmm_fwd_pieces > 1 - the draw reads the
 * pieces' sums: it picks the piece in which their prefix passes the cell's
 * target, then walks that piece's terms).  No counterpart in the reference.
 */
size_t genbmm_samplebmm_stats_size(int B, int M, int K, int N);

/*
 * The same two functions with the kernel family named per call (tests and
 * measurements; the plain functions are GENBMM_PATH_AUTO).
 *   GENBMM_PATH_AUTO   whole-item kernels for matrices up to 64^3, the matrix
 *                      cores where the shape allows (every extent at least
 *                      96, or items of one 128 x 128 tile), else the factored
 *                      kernels on the vector ALU;
 *   GENBMM_PATH_EXACT  the online / exp-per-term kernels only (what a NULL
 *                      `stats` gives; a non-NULL one still receives the maxima);
 *   GENBMM_PATH_VALU   the factored kernels contracting with v_fma_f32 on the
 *                      vector ALU, never the matrix cores or whole-item kernels.
 *   GENBMM_PATH_FACTORS as AUTO, but the matrix-core forward leaves
 *                      exp(a - max), exp(b - max) and 1 / sum in `stats`
 *                      (201 MB at 64 x 512^3) and the matrix-core backward
 *                      reads them instead of forming them again: a backward
 *                      without an exponential, at 600 times the workspace.
 * Under AUTO the matrix-core kernels keep the reference's memory footprint (it
 * saves one `maxes` tensor, genmul.py:29-32): `stats` holds the row / column
 * maxima and a flag per tile (0.3 MB at 64 x 512^3), and the backward forms
 * exp(a - max), exp(b - max) and g exp(max - out) again while it stages them -
 * measured 3 % faster per forward + backward than keeping the factors (the
 * forward writes 200 MB less, the backward takes three exponentials per staged
 * element).  With float16 / bfloat16 tensors that backward reads `out` as stored
 * (rounded); FACTORS keeps 1 / sum in fp32.
 *   GENBMM_PATH_MFMA32 as AUTO, but the matrix-core kernels use the fp32 matrix
 *                      instruction.  Under AUTO they run on the bf16 matrix
 *                      instruction with every factor cut into three bf16
 *                      parts that add up to it exactly and six partial
 *                      products per product, accumulated in fp32 - what is
 *                      dropped is below 2^-23 of a product, one fp32 rounding -
 *                      at 2.7 times less matrix-pipe time (the forward for any
 *                      sizes; the backward where K and N are multiples of 4,
 *                      else it stays on the fp32 instruction).
 * Any other value: GENBMM_E_MODE.  Forward and backward of one problem need not
 * name the same path (see genbmm_logbmm_bwd).  No counterpart in the reference.
 */
#define GENBMM_PATH_AUTO 0
#define GENBMM_PATH_EXACT 1
#define GENBMM_PATH_VALU 2
#define GENBMM_PATH_FACTORS 3
#define GENBMM_PATH_MFMA32 4
/* Number of fp32 elements of `stats` for a forward / backward pair on `path`
 * (genbmm_logbmm_stats_size is this for GENBMM_PATH_AUTO). */
size_t genbmm_logbmm_stats_size_path(int B, int M, int K, int N, int path);
int genbmm_logbmm_fwd_path(const float* a, const float* b, float* out,
                           float* stats, int B, int M, int K, int N, int path,
                           void* stream);
int genbmm_logbmm_bwd_path(const float* a, const float* b, const float* out,
                           const float* g, const float* stats,
                           float* grad_a, float* grad_b,
                           int B, int M, int K, int N, int path, void* stream);

/*
 * Into how many pieces genbmm_logbmm_fwd (path GENBMM_PATH_AUTO, and its _f16 /
 * _bf16 forms) cuts the reduction axis of this problem: 1 (it does not) unless
 * the result has fewer than 128 tiles of 128 x 128 and K is at least 2048 -
 * every output tile belongs to one workgroup that walks all of K, and such a
 * problem would run on a few of the chip's 256 compute units.  The pieces'
 * sums are added in the workspace (genbmm_logbmm_stats_size counts the room)
 * before the guard is tested and the logarithm taken, so the result is the
 * unsplit one up to the order of the additions.  No counterpart in the
 * reference, whose kernel gives every output cell one thread that walks all
 * of K (matmul_cuda_kernel.cu:13-45).  genbmm_logbmm_fwd_static never cuts.
 */
int genbmm_logbmm_fwd_pieces(int B, int M, int K, int N);

/*
 * genbmm_logbmm_fwd for callers that cannot allocate device memory - code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  It
 * has no counterpart in the reference.  The workspace that genbmm_logbmm_fwd takes
 * as `stats` is a fixed array inside the library instead (4 MiB, one copy on every
 * GPU the library runs on, held until the process ends), and nothing is kept for a
 * backward: this is a forward for its own sake, on the same kernels, with results
 * identical to genbmm_logbmm_fwd's (a problem that genbmm_logbmm_fwd cuts into
 * pieces, genbmm_logbmm_fwd_pieces > 1, runs uncut here: equal up to the order
 * of the additions, and slower).  No hipMalloc / hipFree inside, ever.
 * Limit: B*(M+N) + B*ceil(M/32)*ceil(N/32) + 8 <= genbmm_logbmm_static_limit()
 * (= 1048576 floats; the headline 64 x 512^3 needs 81928); beyond it the call
 * returns GENBMM_E_TOOBIG and does nothing.
 * Every call on a GPU uses that GPU's one array: calls that overlap in time on the
 * same GPU (two streams, two threads) race on it - serialise them.  Nothing in the
 * array needs clearing between calls (each call writes what it reads).  The first
 * call on a device looks the array's address up (hipGetSymbolAddress, no stream
 * work); make that call before starting a graph capture.
 */
int genbmm_logbmm_fwd_static(const float* a, const float* b, float* out,
                             int B, int M, int K, int N, void* stream);
size_t genbmm_logbmm_static_limit(void);

/*
 * Second-order terms of logbmm: the gradients with respect to (a, b, g) of
 * <u_a, grad_a> + <u_b, grad_b> where (grad_a, grad_b) are the outputs of
 * genbmm_logbmm_bwd.  u_a or u_b may be NULL (treated as zeros), not both.
 * With u_b == NULL this is _genbmm.backbackward(a, b, g, out, maxes, u_a, 0):
 * matmul_cuda.cpp:94-109, matmul_cuda_kernel.cu:547-622, kernels :220-331.
 */
int genbmm_logbmm_bwdbwd(const float* a, const float* b, const float* out,
                         const float* g, const float* u_a, const float* u_b,
                         float* grad_a, float* grad_b, float* grad_g,
                         int B, int M, int K, int N, void* stream);

/*
 * The same function on a caller-allocated workspace of
 * genbmm_logbmm_bwdbwd_ws_size(B, M, K, N) floats (NULL: as the function above).
 * With it, problems whose extents are all at least 64 take the factored form on
 * the matrix cores: with EA = exp(a - rowmax), EB = exp(b - colmax),
 * R = exp(rowmax + colmax - out), H = g R, X = EA u_a, Y = EB u_b:
 *   grad_g = t = R (X EB + EA Y),
 *   grad_a = X (H EB^T) + EA (H Y^T - (H t) EB^T),
 *   grad_b = Y (EA^T H) + EB (X^T H - EA^T (H t))
 * - eight batched matrix products (five without u_b) instead of one
 * exponential per (m, k, n) in each of three passes.  Batch items with a cell
 * whose rowmax + colmax - out exceeds 40 ln 2 or is not finite are redone by
 * the exact passes.  Same reference counterpart as genbmm_logbmm_bwdbwd; the
 * workspace is scratch (nothing in it outlives the call).
 */
size_t genbmm_logbmm_bwdbwd_ws_size(int B, int M, int K, int N);
int genbmm_logbmm_bwdbwd_ws(const float* a, const float* b, const float* out,
                            const float* g, const float* u_a, const float* u_b,
                            float* grad_a, float* grad_b, float* grad_g,
                            float* workspace, int B, int M, int K, int N,
                            void* stream);

/*
 * out[b,m,n] = max_k (a[m,k] + b[k,n]); idx = the k attaining it.
 * Ascending k, strict '>' against a running maximum that starts at -1e9
 * with index -1: ties resolve to the lowest k.
 * Replaces _genbmm.forward(a, b, 1): matmul_cuda_kernel.cu:498-511,
 * kernel :47-75.
 */
int genbmm_maxbmm_fwd(const float* a, const float* b, float* out, int32_t* idx,
                      int B, int M, int K, int N, void* stream);

/*
 * Into how many pieces genbmm_maxbmm_fwd and genbmm_prodmaxbmm_fwd (float
 * operands) cut the reduction axis of this problem: 1 (they do not) unless the
 * result has fewer than 128 tiles of 64 x 64 and K is at least 2048.  The
 * pieces' maxima meet in `out` and the lowest k that attains them in `idx` by
 * integer atomics, which commute: values and indices are those of the uncut
 * walk, bit for bit, whatever order the pieces arrive in.  No counterpart in
 * the reference, whose kernel gives every output cell one thread that walks
 * all of K (matmul_cuda_kernel.cu:47-75, :124-152).
 */
int genbmm_maxbmm_fwd_pieces(int B, int M, int K, int N);

/*
 * out[b,m,n] = max_k (a[m,k] * b[k,n]); idx as above.
 * factors (optional, may be NULL): 2*B*M*N floats of workspace for
 * genbmm_prodmax_bwd; receives a[m, idx[m,n]] for every cell, then
 * b[idx[m,n], n] for every cell (0 where idx is -1; nothing when K = 0), so
 * that the backward reads its factors in order instead of gathering them.
 * Replaces _genbmm.forward(a, b, 3): matmul_cuda_kernel.cu:527-541,
 * kernel :124-152.
 */
int genbmm_prodmaxbmm_fwd(const float* a, const float* b, float* out,
                          int32_t* idx, float* factors, int B, int M, int K,
                          int N, void* stream);

/*
 * out = log-sum-exp as genbmm_logbmm_fwd; idx[b,m,n] ~ Categorical(softmax_k
 * (a[m,k] + b[k,n])) by inverse CDF in ascending k against one uniform per
 * output cell.  The uniform of cell i = (b*M + m)*N + n is
 * (x >> 8) * 2^-24 with x = word (i & 3) of Philox4x32-10(counter = {lo32(i >> 2),
 * hi32(i >> 2), lo32(offset), hi32(offset)}, key = {lo32(seed), hi32(seed)}):
 * four consecutive cells share one Philox block.
 * A cell without any mass (every term masked) keeps index 0, as in the
 * reference.  A uniform within rounding of 1 never falls past the last term:
 * the exact walk then names the last term that has mass, and the walks on the
 * factors shrink every target by 2^-22 (matrix cores) or 2^-17 (vector ALU) of
 * itself - where the reference's own scan can run out and leave index 0.
 * Replaces _genbmm.forward(a, b, 2): matmul_cuda_kernel.cu:512-526
 * (torch::rand at :517), kernel :77-121.
 * `stats`: NULL, or a buffer of genbmm_samplebmm_stats_size(B,M,K,N) floats, used
 * like that of genbmm_logbmm_fwd; with it the log-sum-exp comes from the logbmm forward and
 * the CDF walk multiplies staged exp(a-max)*exp(b-max) instead of taking one
 * exponential per term (tiles where that is not exact walk the exact way).
 */
int genbmm_samplebmm_fwd(const float* a, const float* b, float* out,
                         int32_t* idx, float* stats,
                         uint64_t seed, uint64_t offset,
                         int B, int M, int K, int N, void* stream);

/*
 * grad_a[b,m,k] = sum_n [k == idx[m,n]] * g[m,n]   (terms added in ascending n)
 * grad_b[b,k,n] = sum_m [k == idx[m,n]] * g[m,n]   (terms added in ascending m)
 * Backward of maxbmm and samplebmm.  Replaces _genbmm.backward(..., 1|2):
 * matmul_cuda_kernel.cu:676-696, kernels :336-395 (which take the index as a
 * float tensor, genmul.py:62-65).
 */
int genbmm_argmax_bwd(const int32_t* idx, const float* g,
                      float* grad_a, float* grad_b,
                      int B, int M, int K, int N, void* stream);

/*
 * grad_a[b,m,k] = sum_n [k == idx[m,n]] * b[k,n] * g[m,n]
 * grad_b[b,k,n] = sum_m [k == idx[m,n]] * a[m,k] * g[m,n]
 * Each term is rounded as a product and then added (no fused multiply-add),
 * in ascending n (resp. m).  factors: NULL, or the workspace filled by
 * genbmm_prodmaxbmm_fwd for these a, b, idx; a and b are then not read (and may
 * be NULL) and the results are the same bit for bit.  Replaces
 * _genbmm.backward(..., 3): matmul_cuda_kernel.cu:697-718, kernels :399-456.
 */
int genbmm_prodmax_bwd(const float* a, const float* b, const int32_t* idx,
                       const float* factors, const float* g, float* grad_a,
                       float* grad_b, int B, int M, int K, int N, void* stream);

/* ----------------------------------------------------------------- banded */

/*
 * Banded product of a (B, n, a_lu+a_ld+1) with b (B, n, b_lu+b_ld+1) in band
 * storage; the result has lu = a_lu + b_ld, ld = a_ld + b_lu and shape
 * (B, n, Wo), Wo = (a_lu+a_ld+1) + (b_lu+b_ld+1) - 1.  In dense terms the
 * result is  Dense(b)^T (x) Dense(a)  in the chosen semiring.
 *   out[i,j] = (+)_k a[i,k] (x) b[o,k2],  o = i + j - lu_out,
 *              k2 = k - j + (b_lu + b_ld),  0 <= i+k-a_lu < n.
 * mode GENBMM_BAND_LOG: log-sum-exp; GENBMM_BAND_MAX: max-plus, idx (B,n,Wo)
 * receives the arg-max k (index into a's band; -1e9 floor, strict '>');
 * GENBMM_BAND_MUL: ordinary (+,*).  Cells with o outside [0,n) are written
 * as 0 (idx 0).  idx may be NULL unless mode is GENBMM_BAND_MAX.
 * `workspace`: NULL, or (used in mode LOG only) a buffer of
 * genbmm_banded_workspace_size floats.  With it the forward takes every
 * exponential once - exp(a - rowmax), exp(b - rowmax) in a pass of its own,
 * kept together with the maxima and 1/sum per output cell - and
 * genbmm_banded_bwd, handed the same buffer, takes none.  It stands where the
 * reference's `maxes` output stands.
 * Replaces _genbmm.forward_band: matmul_cuda.cpp:112-124,
 * banded_cuda_kernel.cu:354-402, kernel :13-100.
 */
int genbmm_banded_fwd(const float* a, int a_lu, int a_ld,
                      const float* b, int b_lu, int b_ld,
                      float* out, int32_t* idx, float* workspace,
                      int B, int n, int mode, void* stream);

/*
 * Banded sample product: out = the log product (mode GENBMM_BAND_LOG above),
 * idx[i,j] = one term k of the cell (index into a's band, as mode MAX stores
 * its arg-max) drawn with probability exp(a[i,k] + b[o,k2] - out[i,j]).  The
 * reference's band kernel has modes 0, 1 and 3 only
 * (banded_cuda_kernel.cu:42, 65, 76); this is its dense sampling rule
 * (sample_cuda_forward_kernel, matmul_cuda_kernel.cu:107-118: ascending
 * terms, the first with total < r && total + p > r) applied to a band cell's
 * terms, with r the Philox4x32-10 uniform of the cell's linear index for
 * (seed, offset), exactly as genbmm_samplebmm_fwd draws it.  A cell whose walk
 * never brackets r keeps its first term; cells outside the matrix get 0.
 * `workspace`: NULL or genbmm_banded_workspace_size floats (then the walk runs
 * on the log product's factors and takes no exponential).  The gradients are
 * genbmm_banded_bwd's with mode GENBMM_BAND_SAMPLE (one-hot scatter of g, as
 * the dense sample op uses the arg-max backward, matmul_cuda_kernel.cu:676).
 */
int genbmm_banded_sample_fwd(const float* a, int a_lu, int a_ld,
                             const float* b, int b_lu, int b_ld,
                             float* out, int32_t* idx, float* workspace,
                             uint64_t seed, uint64_t offset,
                             int B, int n, void* stream);

/* Number of fp32 elements of the log product's workspace (0 on bad arguments). */
size_t genbmm_banded_workspace_size(int a_lu, int a_ld, int b_lu, int b_ld,
                                    int B, int n);

/*
 * 1 if the (+,x) and log products of these bands, forward and backward, run on
 * the kernels that feed the matrix cores (from 3 diagonals per operand up to
 * about 225); 0 if they fall to one lane per result cell, which is 20 to 40
 * times slower per cell - a caller whose matrices are small may then prefer
 * dense algebra (the host layer does: to_dense, the dense product, banddiag).
 * No counterpart in the reference, which has the one kernel for every width.
 */
int genbmm_banded_on_matrix_cores(int a_lu, int a_ld, int b_lu, int b_ld,
                                  int B, int n);

/*
 * Gradients of genbmm_banded_fwd with respect to BOTH operands, reading g,
 * out and idx in the frame the forward wrote them (no banded transposes).
 * `out` is read in mode LOG only, `idx` in mode MAX only (others may be NULL);
 * `workspace`: NULL or, in mode LOG, the buffer the forward filled; the backward
 * writes its own part of it (g/S per output cell, shared by both gradients), so
 * two backward calls on one workspace must not overlap in time.
 * grad_a terms are added in ascending j (result band index), grad_b terms in
 * ascending i (row of a), which is the order of the reference's two calls.
 * Replaces the two _genbmm.backward_band calls and the Python-side banded
 * transposes of BandedMul / BandedLogMul / BandedMaxMul.backward
 * (sparse.py:404-447, 466-545, 579-637; matmul_cuda.cpp:126-143;
 * banded_cuda_kernel.cu:404-450, kernel :104-152).
 */
int genbmm_banded_bwd(const float* a, int a_lu, int a_ld,
                      const float* b, int b_lu, int b_ld,
                      const float* out, const int32_t* idx,
                      float* workspace, const float* g,
                      float* grad_a, float* grad_b,
                      int B, int n, int mode, void* stream);

/*
 * Floats that genbmm_banded_bwd_scratch needs in `scratch` for a log product of these
 * bands; 0 where the backward keeps nothing beside the workspace (the kernels that
 * form g/S while they read g: from 3 diagonals per operand up to about 160 in the
 * result).  No counterpart in the reference, which allocates its temporaries itself.
 */
size_t genbmm_banded_scratch_size(int a_lu, int a_ld, int b_lu, int b_ld,
                                  int B, int n);

/*
 * genbmm_banded_bwd with the workspace left untouched: what the backward keeps
 * beside it (g/S per output cell, mode LOG with a workspace only) goes to
 * `scratch`, genbmm_banded_scratch_size floats, which must be given whenever
 * `workspace` is and that size is not 0.
 * For callers that must not write to what the forward returned - operator
 * frameworks that check their inputs for mutation, or several backward calls
 * on one workspace at a time, each with a scratch buffer of its own.  Same
 * reference counterpart as genbmm_banded_bwd.
 */
int genbmm_banded_bwd_scratch(const float* a, int a_lu, int a_ld,
                              const float* b, int b_lu, int b_ld,
                              const float* out, const int32_t* idx,
                              const float* workspace, float* scratch,
                              const float* g, float* grad_a, float* grad_b,
                              int B, int n, int mode, void* stream);

/*
 * Log-semiring second-order terms: gradients with respect to (a, b, g) of
 * <u_a, grad_a> + <u_b, grad_b> for the outputs of genbmm_banded_bwd in mode
 * LOG.  u_a or u_b may be NULL (zeros), not both.
 * Replaces _genbmm.backbackward_band: matmul_cuda.cpp:145-161,
 * banded_cuda_kernel.cu:453-546, kernels :154-350.
 */
int genbmm_banded_bwdbwd(const float* a, int a_lu, int a_ld,
                         const float* b, int b_lu, int b_ld,
                         const float* out, const float* g,
                         const float* u_a, const float* u_b,
                         float* grad_a, float* grad_b, float* grad_g,
                         int B, int n, void* stream);

/* ------------------------------------------------- band storage, structure */

/*
 * The reference has no native entry points for these: genbmm/sparse.py builds
 * them from torch cat / flip / unfold / diagonal / contiguous calls on the band
 * tensor.  Each one below is a single pass (one read, one write).  data is
 * (B, n, W = lu + ld + 1), data[b, c, k] = Dense[b, c + k - lu, c].
 */

/*
 * out[b, c, k] = data[b, c + dcol, k + dband] where that lies inside
 * (n, w_in), else fill; out is (B, n, w_out).  With the band offsets
 * re-labelled by the caller this is band_shift(t) (dband = t, sparse.py:96-110),
 * band_pad(t) (dband = -|t|, w_out = w_in + 2|t|, :112-123), band_unshift
 * (dband = -1, :137-152), col_shift(t) (dcol = t, :154-165), col_unshift
 * (dcol = -1, :167-182) and _expand (dband = -(lu' - lu), :192-197).
 */
int genbmm_band_shift(const float* data, float* out, int B, int n, int w_in,
                      int w_out, int dcol, int dband, float fill, void* stream);

/*
 * Element-wise op on the union band (lu = max(a_lu, b_lu), ld = max(a_ld,
 * b_ld)): out = zero; out[a's cells] = a; out[b's cells] = op(out, b), as
 * BandedMatrix.op does (sparse.py:199-212).
 */
#define GENBMM_OP_ADD 0
#define GENBMM_OP_MUL 1
#define GENBMM_OP_MAX 2
#define GENBMM_OP_MIN 3
int genbmm_band_op(const float* a, int a_lu, int a_ld,
                   const float* b, int b_lu, int b_ld, float* out,
                   int B, int n, int op, float zero, void* stream);

/*
 * Band storage of the transposed matrix (its lu is ld, its ld is lu):
 * out[b, c, k] = data[b, c + k - ld, W - 1 - k], 0 where that row does not
 * exist (Transpose / repdiag and BandedMatrix.transpose, sparse.py:33-77,
 * 214-218).
 */
int genbmm_band_transpose(const float* data, float* out, int B, int n,
                          int lu, int ld, void* stream);

/*
 * out (B, n, n): out[b, r, c] = data[b, c, r - c + lu] inside the band, else
 * fill (BandedMatrix.to_dense, sparse.py:184-190).
 */
int genbmm_band_to_dense(const float* data, float* out, int B, int n,
                         int lu, int ld, float fill, void* stream);

/*
 * Band storage of dense (B, n_rows, n): out[b, c, k] = dense[b, c + k - lu, c],
 * 0 where that row does not exist (banddiag, sparse.py:12-30).
 */
int genbmm_band_from_dense(const float* dense, float* out, int B, int n_rows,
                           int n, int lu, int ld, void* stream);

/* ------------------------------------------------------- double precision */

/*
 * The reference instantiates all of its kernels for double as well
 * (AT_DISPATCH_FLOATING_TYPES_AND_HALF, matmul_cuda_kernel.cu:489 and on,
 * banded_cuda_kernel.cu:389 and on).  The functions below are the same
 * operations as their float namesakes above on double buffers, with the same
 * argument meaning and return codes, minus the float path's workspaces
 * (stats / factors / workspace).  logbmm forward and backward run factored on
 * the double-precision matrix instruction (64 x 64 tiles; row and column
 * maxima, exponentials and the guard S >= 1e-280 inside the one kernel, cells
 * that fail it redone by the reference's own two passes) for problems of at
 * least 4096 terms with M, N <= 4096; everything else is one lane per result
 * cell, the reduction walked in ascending order as the reference does.
 * samplebmm draws the same uniform (24 random bits) per cell as the float
 * function for a given seed and offset.
 */
int genbmm_logbmm_fwd_f64(const double* a, const double* b, double* out,
                          int B, int M, int K, int N, void* stream);
int genbmm_logbmm_bwd_f64(const double* a, const double* b, const double* out,
                          const double* g, double* grad_a, double* grad_b,
                          int B, int M, int K, int N, void* stream);
int genbmm_logbmm_bwdbwd_f64(const double* a, const double* b, const double* out,
                             const double* g, const double* u_a, const double* u_b,
                             double* grad_a, double* grad_b, double* grad_g,
                             int B, int M, int K, int N, void* stream);
int genbmm_maxbmm_fwd_f64(const double* a, const double* b, double* out,
                          int32_t* idx, int B, int M, int K, int N, void* stream);
int genbmm_prodmaxbmm_fwd_f64(const double* a, const double* b, double* out,
                              int32_t* idx, int B, int M, int K, int N,
                              void* stream);
int genbmm_samplebmm_fwd_f64(const double* a, const double* b, double* out,
                             int32_t* idx, uint64_t seed, uint64_t offset,
                             int B, int M, int K, int N, void* stream);
int genbmm_argmax_bwd_f64(const int32_t* idx, const double* g, double* grad_a,
                          double* grad_b, int B, int M, int K, int N,
                          void* stream);
int genbmm_prodmax_bwd_f64(const double* a, const double* b, const int32_t* idx,
                           const double* g, double* grad_a, double* grad_b,
                           int B, int M, int K, int N, void* stream);
int genbmm_banded_fwd_f64(const double* a, int a_lu, int a_ld,
                          const double* b, int b_lu, int b_ld,
                          double* out, int32_t* idx,
                          int B, int n, int mode, void* stream);
int genbmm_banded_sample_fwd_f64(const double* a, int a_lu, int a_ld,
                                 const double* b, int b_lu, int b_ld,
                                 double* out, int32_t* idx,
                                 uint64_t seed, uint64_t offset,
                                 int B, int n, void* stream);
int genbmm_banded_bwd_f64(const double* a, int a_lu, int a_ld,
                          const double* b, int b_lu, int b_ld,
                          const double* out, const int32_t* idx, const double* g,
                          double* grad_a, double* grad_b,
                          int B, int n, int mode, void* stream);
int genbmm_banded_bwdbwd_f64(const double* a, int a_lu, int a_ld,
                             const double* b, int b_lu, int b_ld,
                             const double* out, const double* g,
                             const double* u_a, const double* u_b,
                             double* grad_a, double* grad_b, double* grad_g,
                             int B, int n, void* stream);

/* --------------------------------------------------------- half precision */

/*
 * The reference instantiates its dense kernels for Half too
 * (AT_DISPATCH_FLOATING_TYPES_AND_HALF, matmul_cuda_kernel.cu:489, :503, :518,
 * :533 for the four forwards, :654-:709 for the backwards), computing in
 * scalar_t = Half.
 * The functions below are the float functions of the same name compiled for
 * tensors of IEEE binary16 (`_f16`) and bfloat16 (`_bf16`) elements, passed as
 * their 16-bit patterns: a, b, out, g, grad_a and grad_b are of that type;
 * stats, factors and idx keep their float / int32 types and the sizes the float
 * functions use (genbmm_logbmm_stats_size, genbmm_samplebmm_stats_size,
 * 2*B*M*N factors).  A value is widened by the load that fetches it, all
 * arithmetic and every workspace is fp32, a result is rounded to nearest-even
 * by the store that writes it: each function returns exactly what its float
 * namesake returns on the widened tensors, rounded once (indices: identical).
 * The backward functions that read `out` read the rounded one, as the
 * reference's do.  samplebmm sweeps only where the forward left 1/S in the
 * workspace (matrix-core shapes, K <= 2016) and walks the terms exactly
 * otherwise (`out` rounded to 11 or 8 bits does not give S well enough for the
 * other sweeps): its index is the float function's on those shapes and the
 * index of the float function called with stats = NULL on all others.
 * The second-order function exists in its workspace form only
 * (genbmm_logbmm_bwdbwd_ws_f16 / _bf16; the workspace is required: the gradient
 * with respect to g is read back by the other two and stays unrounded there).
 * The banded functions likewise (the reference instantiates every banded kernel
 * for Half too, banded_cuda_kernel.cu:389, :435, :484, :508, :530): band data,
 * results, g and gradients in the 16-bit type, `workspace` and `scratch` float
 * with the sizes of the float functions.  The second-order function takes one
 * more buffer, `t_scratch` (B * n * Wo floats): the gradient with respect to g
 * is read back by the other two gradients and must stay unrounded there
 * (grad_g receives it rounded).
 */
int genbmm_logbmm_fwd_f16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                          float* stats, int B, int M, int K, int N, void* stream);
int genbmm_logbmm_fwd_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                           float* stats, int B, int M, int K, int N, void* stream);
int genbmm_logbmm_bwd_f16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                          const uint16_t* g, const float* stats,
                          uint16_t* grad_a, uint16_t* grad_b,
                          int B, int M, int K, int N, void* stream);
int genbmm_logbmm_bwd_bf16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                           const uint16_t* g, const float* stats,
                           uint16_t* grad_a, uint16_t* grad_b,
                           int B, int M, int K, int N, void* stream);
int genbmm_logbmm_fwd_path_f16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                               float* stats, int B, int M, int K, int N, int path,
                               void* stream);
int genbmm_logbmm_fwd_path_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                                float* stats, int B, int M, int K, int N, int path,
                                void* stream);
int genbmm_logbmm_bwd_path_f16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                               const uint16_t* g, const float* stats,
                               uint16_t* grad_a, uint16_t* grad_b,
                               int B, int M, int K, int N, int path, void* stream);
int genbmm_logbmm_bwd_path_bf16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                                const uint16_t* g, const float* stats,
                                uint16_t* grad_a, uint16_t* grad_b,
                                int B, int M, int K, int N, int path, void* stream);
int genbmm_maxbmm_fwd_f16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                          int32_t* idx, int B, int M, int K, int N, void* stream);
int genbmm_maxbmm_fwd_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                           int32_t* idx, int B, int M, int K, int N, void* stream);
int genbmm_prodmaxbmm_fwd_f16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                              int32_t* idx, float* factors,
                              int B, int M, int K, int N, void* stream);
int genbmm_prodmaxbmm_fwd_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                               int32_t* idx, float* factors,
                               int B, int M, int K, int N, void* stream);
int genbmm_samplebmm_fwd_f16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                             int32_t* idx, float* stats, uint64_t seed, uint64_t offset,
                             int B, int M, int K, int N, void* stream);
int genbmm_samplebmm_fwd_bf16(const uint16_t* a, const uint16_t* b, uint16_t* out,
                              int32_t* idx, float* stats, uint64_t seed, uint64_t offset,
                              int B, int M, int K, int N, void* stream);
int genbmm_argmax_bwd_f16(const int32_t* idx, const uint16_t* g,
                          uint16_t* grad_a, uint16_t* grad_b,
                          int B, int M, int K, int N, void* stream);
int genbmm_argmax_bwd_bf16(const int32_t* idx, const uint16_t* g,
                           uint16_t* grad_a, uint16_t* grad_b,
                           int B, int M, int K, int N, void* stream);
int genbmm_prodmax_bwd_f16(const uint16_t* a, const uint16_t* b, const int32_t* idx,
                           const float* factors, const uint16_t* g,
                           uint16_t* grad_a, uint16_t* grad_b,
                           int B, int M, int K, int N, void* stream);
int genbmm_prodmax_bwd_bf16(const uint16_t* a, const uint16_t* b, const int32_t* idx,
                            const float* factors, const uint16_t* g,
                            uint16_t* grad_a, uint16_t* grad_b,
                            int B, int M, int K, int N, void* stream);

int genbmm_logbmm_bwdbwd_ws_f16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                                const uint16_t* g, const uint16_t* u_a, const uint16_t* u_b,
                                uint16_t* grad_a, uint16_t* grad_b, uint16_t* grad_g,
                                float* workspace, int B, int M, int K, int N,
                                void* stream);
int genbmm_logbmm_bwdbwd_ws_bf16(const uint16_t* a, const uint16_t* b, const uint16_t* out,
                                 const uint16_t* g, const uint16_t* u_a, const uint16_t* u_b,
                                 uint16_t* grad_a, uint16_t* grad_b, uint16_t* grad_g,
                                 float* workspace, int B, int M, int K, int N,
                                 void* stream);
int genbmm_banded_fwd_f16(const uint16_t* a, int a_lu, int a_ld,
                          const uint16_t* b, int b_lu, int b_ld,
                          uint16_t* out, int32_t* idx, float* workspace,
                          int B, int n, int mode, void* stream);
int genbmm_banded_sample_fwd_f16(const uint16_t* a, int a_lu, int a_ld,
                                 const uint16_t* b, int b_lu, int b_ld,
                                 uint16_t* out, int32_t* idx, float* workspace,
                                 uint64_t seed, uint64_t offset,
                                 int B, int n, void* stream);
int genbmm_banded_bwd_f16(const uint16_t* a, int a_lu, int a_ld,
                          const uint16_t* b, int b_lu, int b_ld,
                          const uint16_t* out, const int32_t* idx,
                          float* workspace, const uint16_t* g,
                          uint16_t* grad_a, uint16_t* grad_b,
                          int B, int n, int mode, void* stream);
int genbmm_banded_bwd_scratch_f16(const uint16_t* a, int a_lu, int a_ld,
                                  const uint16_t* b, int b_lu, int b_ld,
                                  const uint16_t* out, const int32_t* idx,
                                  const float* workspace, float* scratch,
                                  const uint16_t* g, uint16_t* grad_a, uint16_t* grad_b,
                                  int B, int n, int mode, void* stream);
int genbmm_banded_bwdbwd_f16(const uint16_t* a, int a_lu, int a_ld,
                             const uint16_t* b, int b_lu, int b_ld,
                             const uint16_t* out, const uint16_t* g,
                             const uint16_t* u_a, const uint16_t* u_b,
                             uint16_t* grad_a, uint16_t* grad_b, uint16_t* grad_g,
                             float* t_scratch, int B, int n, void* stream);
int genbmm_banded_fwd_bf16(const uint16_t* a, int a_lu, int a_ld,
                          const uint16_t* b, int b_lu, int b_ld,
                          uint16_t* out, int32_t* idx, float* workspace,
                          int B, int n, int mode, void* stream);
int genbmm_banded_sample_fwd_bf16(const uint16_t* a, int a_lu, int a_ld,
                                 const uint16_t* b, int b_lu, int b_ld,
                                 uint16_t* out, int32_t* idx, float* workspace,
                                 uint64_t seed, uint64_t offset,
                                 int B, int n, void* stream);
int genbmm_banded_bwd_bf16(const uint16_t* a, int a_lu, int a_ld,
                          const uint16_t* b, int b_lu, int b_ld,
                          const uint16_t* out, const int32_t* idx,
                          float* workspace, const uint16_t* g,
                          uint16_t* grad_a, uint16_t* grad_b,
                          int B, int n, int mode, void* stream);
int genbmm_banded_bwd_scratch_bf16(const uint16_t* a, int a_lu, int a_ld,
                                  const uint16_t* b, int b_lu, int b_ld,
                                  const uint16_t* out, const int32_t* idx,
                                  const float* workspace, float* scratch,
                                  const uint16_t* g, uint16_t* grad_a, uint16_t* grad_b,
                                  int B, int n, int mode, void* stream);
int genbmm_banded_bwdbwd_bf16(const uint16_t* a, int a_lu, int a_ld,
                             const uint16_t* b, int b_lu, int b_ld,
                             const uint16_t* out, const uint16_t* g,
                             const uint16_t* u_a, const uint16_t* u_b,
                             uint16_t* grad_a, uint16_t* grad_b, uint16_t* grad_g,
                             float* t_scratch, int B, int n, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* GENBMM_GFX950_H */
