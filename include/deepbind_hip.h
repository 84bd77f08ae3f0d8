/* deepbind_hip.h - C ABI of libdeepbind_hip.so (gfx950 / MI355X).
 *
 * Every entry point is the raw-pointer form of one of the reference's internal launch
 * functions (the layer its C++ `api_*` exports dispatch to), with
 *   - a hipStream_t (passed as void*) where the reference takes a cudaStream_t,
 *   - an int status return (0 = ok) plus dbk_last_error(), which keeps the reference's
 *     poll-after-every-call convention (reference: smat/py/smat/smat_dll.py:166-183,
 *     smat/src/smat/config.h:95-105),
 *   - device pointers only; no call allocates its outputs (the caller does, as the
 *     reference's Python wrappers do: kangaroo/_ext/kangaroo_smat.py:121-132).
 * Matrices are row-major with full stride; "filter fastest" layouts are the reference's.
 * Calls are asynchronous on `stream`, ordered within it. One process per GPU; a context
 * (device + scratch workspace) must not be shared between host threads without external
 * locking, as in the reference (smat/src/smat/vm/context.cpp:71).
 *
 * All reference paths below are relative to /root/reference/code/libs.
 */
#ifndef DEEPBIND_HIP_H
#define DEEPBIND_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* dbk_stream_t;                 /* hipStream_t */

/* reference: smat/src/smat/dtypes.h (dtype_t); only the two float types reach these ops */
enum { DBK_F32 = 0, DBK_F64 = 1 };

/* reference: kangaroo/kangaroo_smat/kangaroo_smat.h:42-47 (pooltype_t) */
enum { DBK_PT_MAX = 0, DBK_PT_AVG = 1, DBK_PT_SUM = 2, DBK_PT_ALL = 3 };

/* Text of the last failure on the calling thread ("" if none); cleared by the next successful call.
 * reference: api_get_last_error, smat/py/smat/smat_dll.py:166-183 */
const char* dbk_last_error(void);
/* Library/ABI version, bumped when a signature changes. */
int dbk_version(void);
/* Number of HIP devices visible; <0 on failure. Touches the runtime only to count devices. */
int dbk_device_count(void);
/* on != 0: from now on dbk_corr1ord, dbk_corr1ord_bprop_W and dbk_corr1ord_bprop_X keep to their lookup / vector
 * kernels at EVERY size, so that a row's result does not depend on the size of the batch it arrives in: dbk_corr1ord
 * then adds the taps in the reference's order (corr1ord.cuh:139-157: its bits) for any number of rows, and the two
 * gradients keep one summation order. Off (the default) float32 calls switch to the matrix-core kernels at bulk sizes
 * (2^25 map values for the forward, 2^22 for the gradients): the same sums in another order, 1.5-2x faster.
 * Process-wide; returns the previous setting. No counterpart in the reference (it has one kernel per operator). */
int dbk_set_exact_scan(int on);
/* Blocks until `stream` has drained. reference: api_sync, smat_cuda/cuda_context.cpp:198-202 */
int dbk_sync(dbk_stream_t stream);

/* ------------------------------------------------------------------ motif scan (corr1ord) */

/* Z[i,f] = sum_{j<m} w(j, X[i+j], f) for i < n, where w = W[(C*j+k)*F+f] for k<C, 0 for k==254,
 * and the channel mean for any other code (255 = N / padding). n = number of outputs written
 * (N-m+1); rows >= n of Z are left untouched. W is (C*m, F), X has n+m-1 bytes, Z is (>=n, F).
 * The taps are added in ascending order (the reference's bits) except for float32 maps of 2^25 values or more, which
 * the matrix cores compute (filters of up to 32 taps, at least 32 filters): the same sums in another order.
 * reference: launch_corr1ord, kangaroo/kangaroo_smat/kangaroo_smat.cpp:43-46, corr1ord.cu:136-148 */
int dbk_corr1ord(dbk_stream_t stream, int dtype,
                 const void* W, size_t m, size_t nfilter,
                 const uint8_t* X, size_t n, size_t nchannel,
                 void* Z);

/* dW[(C*j+k),f] += sum_{i<n} dZ[i,f] * [X[i+j]==k]; N/pad codes add dZ/C to all C rows, 254 nothing.
 * Deterministic: per-workgroup private accumulators and a fixed-order reduction, no float atomics (from 4 M
 * float32 gradient values on the matrix cores form the partial sums: another fixed order).
 * reference: launch_corr1ord_bprop_W, kangaroo_smat.cpp:48-51, corr1ord_bprop.cu:97-108 */
int dbk_corr1ord_bprop_W(dbk_stream_t stream, int dtype,
                         void* dW, size_t m, size_t nfilter,
                         const uint8_t* X, size_t n, size_t nchannel,
                         const void* dZ);

/* dX[i,c] += sum_f sum_{k<m, k<=i} dZ[i-k,f] * W[(C*k+c),f] for i < n; dX is (n, C), dZ is (n, F).
 * Computed on the device (the reference copies to the host and loops there); from 4 M float32 gradient values on as a
 * product on the matrix cores (both operands in exact bf16 pieces): the same sums in another order.
 * reference: launch_corr1ord_bprop_X, kangaroo_smat.cpp:53-56, corr1ord_bprop.cu:167-224 */
int dbk_corr1ord_bprop_X(dbk_stream_t stream, int dtype,
                         void* dX, size_t n, size_t nchannel,
                         const void* W, size_t m, size_t nfilter,
                         const void* dZ);

/* ------------------------------------------------------------------ region pooling (poolrgn) */

/* Per region r = [R[r,0], R[r,1]) (optional third column = row step) and column f:
 * max (first strict maximum, argmax = row*F+f as uint32), avg, sum, or all = (max,avg) interleaved
 * at columns (2f, 2f+1). pooled is (P, F) or (P, 2F); argmax may be NULL.
 * reference: launch_poolrgn, kangaroo_smat.cpp:71-74, poolrgn.cu:56-68 */
int dbk_poolrgn(dbk_stream_t stream, int dtype,
                const void* unpooledmaps, size_t nfeaturemap,
                const uint32_t* regions, size_t nregion, int per_region_step,
                void* pooledmaps, uint32_t* pooledmaps_argmax, int ptype);

/* Accumulates into unpooledmaps (N, F): max adds pooled[r,f] at argmax[r,f]; avg/sum spread
 * pooled[r,f](/count) over the region's rows; all does both from the interleaved pairs.
 * Bit-reproducible whenever regions do not overlap (each element then has one writer).
 * reference: launch_poolrgn_bprop, kangaroo_smat.cpp:76-79, poolrgn_bprop.cu:60-72 */
int dbk_poolrgn_bprop(dbk_stream_t stream, int dtype,
                      void* unpooledmaps, size_t nfeaturemap,
                      const uint32_t* regions, size_t nregion, int per_region_step,
                      const void* pooledmaps, const uint32_t* pooledmaps_argmax, int ptype);

/* Input-base dropout: M = (X == 255) || (u >= rate); Z = M ? X : 254 (padding always passes).
 * u comes from the library's counter-based generator at (seed, offset); when `counter` is not null
 * the offset is read from that device word instead (see dbk_counter_add).
 * reference: launch_dropoutord_fp_tr, kangaroo_smat.cpp:81-82, dropoutord.cu:41-60 */
int dbk_dropoutord_fp_tr(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M, size_t n,
                         float rate, uint64_t seed, uint64_t offset, const uint64_t* counter);
/* Same with caller-supplied uniforms U (n floats) instead of the generator. */
int dbk_dropoutord_fp_tr_u(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M, size_t n,
                           float rate, const float* U);
/* Reverse-complement mode of the input dropout: regions come in (fwd, rev) pairs of equal length,
 * each [padding | sequence]; the reverse strand's mask becomes the forward strand's mask mirrored
 * (letter t <-> letter len-1-t) and Z is rewritten there as M ? X : 254.
 * reference: the host loop in kangaroo/_ext/dropoutord.py:55-68 */
int dbk_dropoutord_mirror(dbk_stream_t stream, const uint8_t* X, uint8_t* Z, uint8_t* M,
                          const uint32_t* regions, size_t nregion, size_t padding);

/* ------------------------------------------------------------------ fused scan + bias + ReLU + pool */

/* pooled[r, .] = pool_{i in region r} relu(scan(W,X)[i,f] + bias[f]) without materialising the
 * (N, F) map. Regions have 2 columns. ptype per call (max / avg / all fused; sum goes through
 * dbk_scanpool_fprop_unfused and writes no activity masks); pooled layout and argmax
 * (flat row*F+f into the virtual map, may be NULL) exactly as dbk_poolrgn. X has N bytes; windows
 * reaching past N contribute nothing (the unfused chain leaves those rows at relu(bias)).
 * float32 only. Replaces the chain corr1ord -> bias -> relu -> poolrgn
 * (reference: kangaroo/_ext/corr1ord.py:97-117, deepity/std/elemwise.py:71-82,162-180,
 *  kangaroo/_ext/poolrgn.py:56-76,153-174).
 * act (may be NULL): N * ceil(nfilter/64) 64-bit words that receive, for every row inside a region and
 * every tile of 64 filters, the mask of filters whose rectifier is open there (bit l = filter tile*64 + l):
 * what the reference's relu node keeps as its output for the backward pass (elemwise.py:78), 1 bit per
 * value. Hand it to dbk_scanpool_bprop and the average-pooling gradient needs no recomputation. With act
 * the general kernel runs (the table kernel does not write it). */
int dbk_scanpool_fprop(dbk_stream_t stream,
                       const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N,
                       const uint32_t* regions, size_t nregion, int ptype,
                       float* pooled, uint32_t* argmax, uint64_t* act);

/* Same contract, always through the general kernel (any filter length that fits in LDS, any letter
 * code); dbk_scanpool_fprop picks a faster kernel when the shape allows and otherwise calls this. */
int dbk_scanpool_fprop_general(dbk_stream_t stream,
                               const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N,
                               const uint32_t* regions, size_t nregion, int ptype,
                               float* pooled, uint32_t* argmax, uint64_t* act);

/* Same contract through the four-filters-per-lane lookup kernel regardless of problem size: one wave per region,
 * filters of 9 to 24 taps (NotImplementedError otherwise). Per position the taps are added in the order of the
 * one-filter-per-lane kernel, so maxima, argmax and activity masks are the same bits; averages add the same values in
 * another order. (For many regions dbk_scanpool_fprop_general picks the matrix-core kernel below, which is faster.) */
int dbk_scanpool_fprop_wide(dbk_stream_t stream,
                            const float* W, const float* bias, size_t m, size_t nfilter,
                            const uint8_t* X, size_t N,
                            const uint32_t* regions, size_t nregion, int ptype,
                            float* pooled, uint32_t* argmax, uint64_t* act);

/* Same contract through the matrix-core kernel regardless of problem size (dbk_scanpool_fprop_general picks it once
 * regions x filter tiles reach 512, for filters of 9 to 32 taps), for filters of up to 32 taps
 * (NotImplementedError otherwise): the scan as a product of the windows' one-hot letters with W, each float32
 * weight entering as three bf16 pieces that add up to it exactly, accumulated in float32 by
 * v_mfma_f32_32x32x16_bf16. The sums are those of the lookup kernels in another order: results agree with them
 * to round-off, not bit for bit (an argmax can move between rows whose values tie to round-off). */
int dbk_scanpool_fprop_mfma(dbk_stream_t stream,
                            const float* W, const float* bias, size_t m, size_t nfilter,
                            const uint8_t* X, size_t N,
                            const uint32_t* regions, size_t nregion, int ptype,
                            float* pooled, uint32_t* argmax, uint64_t* act);

/* Same contract through the 3-mer lookup-table kernel regardless of problem size; fails with
 * NotImplementedError for shapes that kernel does not take (filter length > 24, avg/all pooling,
 * argmax requested). Inputs it cannot express (code 254, regions outside the sequence) are detected
 * on the device and computed by the general kernel inside the same call. */
int dbk_scanpool_fprop_kmer(dbk_stream_t stream,
                            const float* W, const float* bias, size_t m, size_t nfilter,
                            const uint8_t* X, size_t N,
                            const uint32_t* regions, size_t nregion, int ptype,
                            float* pooled, uint32_t* argmax);

/* dbk_scanpool_fprop_kmer for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid allocation): same arguments, same kernels, same results, but the call's
 * scratch (a flag word and one index byte per sequence byte) lies in a buffer that is part of the loaded
 * library instead of a grow-on-demand allocation, so the call never allocates, frees or synchronises.
 * Limit: N <= 64 MiB of sequence bytes per call (ValueError beyond; the buffer's 64.0005 MiB are held on every
 * GPU the library runs on until the process ends). All calls on one GPU share the buffer: calls that overlap
 * on one GPU (different streams, different host threads) race; calls ordered on one stream do not.
 * No counterpart in the reference (its wrappers allocate per call, kangaroo/_ext/kangaroo_smat.py:121-132). */
int dbk_scanpool_fprop_kmer_static(dbk_stream_t stream,
                                   const float* W, const float* bias, size_t m, size_t nfilter,
                                   const uint8_t* X, size_t N,
                                   const uint32_t* regions, size_t nregion, int ptype,
                                   float* pooled, uint32_t* argmax);

/* Backward of the fused chain: given dpooled (same layout as pooled), the forward's pooled and
 * argmax, accumulates dW (C*m, F) += (as corr1ord_bprop_W does; with overwrite != 0 it is written
 * instead, which saves the caller a fill) and writes dbias (1, F) =. Deterministic (no float atomics).
 * act (may be NULL): the activity masks dbk_scanpool_fprop wrote for the same W, bias, X and regions;
 * without them the avg / all gradient recomputes them first (a second forward pass into the stream's scratch
 * at bulk sizes while that takes at most 1 GiB, the map through the letter table otherwise).
 * reference chain: poolrgn_bprop -> relu bprop -> bias bprop -> corr1ord_bprop_W
 * (kangaroo/_ext/poolrgn.py:78-82, deepity/std/elemwise.py:78,172-180, kangaroo/_ext/corr1ord.py:120-138) */
int dbk_scanpool_bprop(dbk_stream_t stream,
                       const float* W, const float* bias, size_t m, size_t nfilter,
                       const uint8_t* X, size_t N,
                       const uint32_t* regions, size_t nregion, int ptype,
                       const float* pooled, const uint32_t* argmax, const float* dpooled,
                       float* dW, float* dbias, int overwrite, const uint64_t* act);

/* The same chain for what the fused kernels do not take: sum pooling and regions with a third column (row step).
 * Runs the library's operator kernels one after another (dbk_corr1ord, bias + rectifier, dbk_poolrgn) with the
 * (N x nfilter) map in the stream's scratch (N * nfilter * 4 bytes, grown on demand), so every value is the one the
 * reference's chain produces: rows whose window passes the end of X hold relu(bias), as there. region_columns is 2 or 3;
 * ptype any of the four. dbk_scanpool_fprop / dbk_scanpool_bprop call these for DBK_PT_SUM.
 * reference: kangaroo/_ext/corr1ord.py:97-117, deepity/std/elemwise.py:71-82,162-180, kangaroo/_ext/poolrgn.py:56-76 */
int dbk_scanpool_fprop_unfused(dbk_stream_t stream,
                               const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N,
                               const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                               float* pooled, uint32_t* argmax);
/* Its backward: recomputes the rectified map, spreads dpooled over it (dbk_poolrgn_bprop), gates it by the rectifier,
 * sums the columns into dbias (=) and accumulates dW (+=, or = with overwrite) with dbk_corr1ord_bprop_W. Two maps of
 * scratch. argmax is read for max / all pooling only.
 * reference: kangaroo/_ext/poolrgn.py:78-82, deepity/std/elemwise.py:78,172-180, kangaroo/_ext/corr1ord.py:120-138 */
int dbk_scanpool_bprop_unfused(dbk_stream_t stream,
                               const float* W, const float* bias, size_t m, size_t nfilter,
                               const uint8_t* X, size_t N,
                               const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                               const uint32_t* argmax, const float* dpooled,
                               float* dW, float* dbias, int overwrite);
/* The two calls above in float64, for callers that run the whole path in double precision as the reference can
 * (every operator there is compiled for both float types, corr1ord.cu:129-133): same arguments, same chain of
 * operator kernels (there is no fused float64 kernel), any pooling type, 2 or 3 region columns.
 * reference: as dbk_scanpool_fprop_unfused / dbk_scanpool_bprop_unfused */
int dbk_scanpool_fprop_f64(dbk_stream_t stream,
                           const double* W, const double* bias, size_t m, size_t nfilter,
                           const uint8_t* X, size_t N,
                           const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                           double* pooled, uint32_t* argmax);
int dbk_scanpool_bprop_f64(dbk_stream_t stream,
                           const double* W, const double* bias, size_t m, size_t nfilter,
                           const uint8_t* X, size_t N,
                           const uint32_t* regions, size_t nregion, int region_columns, int ptype,
                           const uint32_t* argmax, const double* dpooled,
                           double* dW, double* dbias, int overwrite);

/* ------------------------------------------------------------------ dense head (deepity_smat) */

/* Z[:, b*m:(b+1)*m] = X_b . W[b*k:(b+1)*k, :]; X_b = X[:, b*k:(b+1)*k], or all of X (n x k) when
 * broadcast_x. X (n, k*nblock | k), W (k*nblock, m), Z (n, m*nblock).
 * reference: launch_blockwise_dot, deepity/deepity_smat/deepity_smat.cpp:75-77, blockwise_dot.cu:77-105 */
int dbk_blockwise_dot(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k, int broadcast_x,
                      const void* X, const void* W, void* Z);
/* dX[:, b*k:(b+1)*k] = dZ[:, b*m:(b+1)*m] . W[b*k:(b+1)*k, :]^T
 * reference: launch_blockwise_dot_nt, deepity_smat.cpp:79-81, blockwise_dot.cu:110-130 */
int dbk_blockwise_dot_nt(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k,
                         const void* dZ, const void* W, void* dX);
/* dW[b*k:(b+1)*k, :] = X_b^T . dZ[:, b*m:(b+1)*m]
 * reference: launch_blockwise_dot_tn, deepity_smat.cpp:83-85, blockwise_dot.cu:132-153 */
int dbk_blockwise_dot_tn(dbk_stream_t stream, int dtype, int nblock, int n, int m, int k, int broadcast_x,
                         const void* X, const void* dZ, void* dW);
/* "combined" forms: W is (p*nblock, m); this input occupies rows [Xoffset, Xoffset+k) of each
 * model's block of p rows. The forward overwrites Z when Xoffset==0 and adds otherwise.
 * reference: launch_blockwise_dot_combined / _nt_combined / _tn_combined,
 * deepity_smat.cpp:87-100, blockwise_dot.cu:156-260 */
int dbk_blockwise_dot_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset, int Xbroadcast,
                               int n, int m, int k, int p, const void* X, const void* W, void* Z);
int dbk_blockwise_dot_nt_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset,
                                  int n, int m, int k, int p, void* dX, const void* W, const void* dZ);
int dbk_blockwise_dot_tn_combined(dbk_stream_t stream, int dtype, int nblock, int Xoffset, int Xbroadcast,
                                  int n, int m, int k, int p, const void* X, void* dW, const void* dZ);

/* Momentum / Nesterov updates with per-element rate vectors.
 * reference: launch_gradstep{,_nesterov1,_nesterov2}, deepity_smat.cpp:42-52, gradstep.cu:41-72 */
int dbk_gradstep(dbk_stream_t stream, int dtype, size_t n,
                 void* P, const void* dP, const void* drate, void* mP, const void* mrate);
int dbk_gradstep_nesterov1(dbk_stream_t stream, int dtype, size_t n,
                           void* P, const void* mP, const void* mrate);
int dbk_gradstep_nesterov2(dbk_stream_t stream, int dtype, size_t n,
                           void* P, const void* dP, const void* drate, void* mP, const void* mrate);

/* The Nesterov step with the look-ahead kept in a vector L beside the parameters, which saves a launch
 * per step: dbk_gradstep_lookahead sets L = P + mrate*mP (what nesterov1 leaves in P); the gradient is
 * taken at L; dbk_gradstep_nesterov2_lookahead then does mP = mrate*mP - drate*dP, P = L - drate*dP and
 * L = P + mrate*mP for the next step. Same operations in the same order as nesterov1 / nesterov2: the
 * parameters come out bit-identical. (reference: gradstep.cu:41-72) */
int dbk_gradstep_lookahead(dbk_stream_t stream, int dtype, size_t n,
                           void* L, const void* P, const void* mP, const void* mrate);
int dbk_gradstep_nesterov2_lookahead(dbk_stream_t stream, int dtype, size_t n,
                                     void* P, void* L, const void* dP, const void* drate, void* mP, const void* mrate);

/* dst[i] += A[i] * b[(i/k) % m] for i < n.
 * reference: launch_madd_bcast, deepity_smat.cpp:54-56, madd_bcast.cu:41-58 */
int dbk_madd_bcast(dbk_stream_t stream, int dtype, const void* A, const void* b, void* dst,
                   size_t n, size_t m, size_t k);

/* A[i] = M[i] ? A[i] : 0 (NaN-safe). reference: launch_maskout, deepity_smat.cpp:58, maskout.cu:41-50 */
int dbk_maskout(dbk_stream_t stream, int dtype, const uint8_t* M, void* A, size_t n);
/* For each (fwd,rev) row pair of Z (n rows, m cols) set M true at the row holding the larger value
 * (ties: first row); other entries are left as they are (the caller pre-zeroes M).
 * reference: launch_calc_zmask, deepity_smat.cpp:60, maskout.cu:52-67 */
int dbk_calc_zmask(dbk_stream_t stream, int dtype, const void* Z, uint8_t* M, size_t n, size_t m);

/* out[i,c] = max(Z[2i,c], Z[2i+1,c]): the prediction kept from each (fwd, rev) row pair; out is (n/2, m).
 * reference: maskout_revcomp, kangaroo/kangaroo/predict.py:145-164 (done there on the host) */
int dbk_pair_max(dbk_stream_t stream, int dtype, const void* Z, void* out, size_t n, size_t m);

/* Dropout on pooled features with one rate per model: column c of an (n/(m*k), m*k) matrix uses
 * rate[(i/k) % m]. keep = (u >= rate). matchrows gives each (2r, 2r+1) row pair one shared draw.
 * reference: launch_dropout_fp_tr / _fp_te / _bp_tr / _bp_te, deepity_smat.cpp:62-73, dropout.cu:41-180 */
int dbk_dropout_fp_tr(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, uint8_t* M,
                      size_t n, size_t m, size_t k, int matchrows, uint64_t seed, uint64_t offset);
/* Same with caller-supplied uniforms U (float32, one per element; with matchrows row 2r's are used). */
int dbk_dropout_fp_tr_u(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z, uint8_t* M,
                        size_t n, size_t m, size_t k, int matchrows, const float* U);
int dbk_dropout_fp_te(dbk_stream_t stream, int dtype, const void* X, const void* rate, void* Z,
                      size_t n, size_t m, size_t k);
int dbk_dropout_bp_tr(dbk_stream_t stream, int dtype, const void* dZ, const uint8_t* M, void* dX, size_t n);
int dbk_dropout_bp_te(dbk_stream_t stream, int dtype, const void* dZ, const void* rate, void* dX,
                      size_t n, size_t m, size_t k);

/* The uniforms the dropout entry points draw: U[i] in [0,1) for flat element i (with matchrows,
 * pair index i). Philox4x32-10, key = seed, counter = offset + i/4, word i%4, top 24 bits.
 * The reference draws from cuRAND's per-thread XORWOW states (smat_cuda/cuda_context.cpp:210-242),
 * which cannot be reproduced without the CUDA SDK; this generator is the library's own. */
int dbk_uniform_fill(dbk_stream_t stream, float* U, size_t n, uint64_t seed, uint64_t offset);
/* dP[i] += sign(P[i]) * decay[i]: the L1 weight-decay term of every parameter in one pass over the flat
 * parameter vector (decay holds each element's coefficient, zero for biases).
 * reference: madd_bcast(sign(W), decay, k, dW) per weight matrix, deepity/std/full.py:111-119,
 * kangaroo/_ext/corr1ord.py:124-126 */
int dbk_l1_decay(dbk_stream_t stream, int dtype, const void* P, const void* decay, void* dP, size_t n);
/* Standard normal deviates from the same generator (Box-Muller on two Philox streams, one value per
 * element, element i depends only on (seed, offset, i)); used for the initial weights.
 * reference: sm.randn in the parameter set-up, deepity/deepity/sgd.py:337-341 (cuRAND there) */
int dbk_normal_fill(dbk_stream_t stream, int dtype, void* Z, size_t n, uint64_t seed, uint64_t offset);
/* Host-side block function of that generator, for known-answer tests. */
int dbk_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);

/* ------------------------------------------------------------------ the few array ops the bias / relu / loss nodes use */

/* Z = X + b (row vector b broadcast down n rows of m columns).
 * reference: kernel_elemwise_b_* add, smat/src/smat_cuda/elemwise3.cuh:193-198, elemwise3.cu:57 */
int dbk_add_rowvec(dbk_stream_t stream, int dtype, const void* X, const void* b, void* Z, size_t n, size_t m);
/* out[c] = sum_r X[r,c] in row order (bias gradient). reference: smat_cuda/reduce_y.cuh:57-91 */
int dbk_colsum(dbk_stream_t stream, int dtype, const void* X, void* out, size_t n, size_t m);
/* Z = max(0, X). reference: smat_cuda/elemwise3.cu:62 */
int dbk_relu(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n);
/* dX = dZ * sign(Z), sign = (z>0)-(z<0). reference: deepity/std/elemwise.py:78, smat_cuda/elemwise2.cu:42,77 */
int dbk_mul_sign(dbk_stream_t stream, int dtype, const void* dZ, const void* Z, void* dX, size_t n);
/* Z = (x>0)-(x<0) (L1 weight-decay gradient). reference: smat_cuda/elemwise2.cu:42,77 */
int dbk_sign(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n);
/* Z = 1/(1+exp(-X)). reference: smat_cuda/elemwise2.cu:46,68 */
int dbk_logistic(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n);
/* Z = softmax of every group of `group` consecutive elements of X (n elements, row-major, group divides the
 * row length): exp(x - max) / sum. The output node of a model with several columns per output.
 * reference: deepity/std/softmax.py:58-71 (rows split into ngroup * ninst chunks), smat softmax checked by
 * smat/py/smat/tests/unittest.py:601-603 */
int dbk_softmax(dbk_stream_t stream, int dtype, const void* X, void* Z, size_t n, size_t group);
/* Elementwise loss terms L (n rows, m cols): kind 0 = log(max(1e-15,Z))*Y + log(max(1e-15,1-Z))*(1-Y),
 * kind 1 = (Z-Y)^2, kind 2 = log(max(1e-15,Z))*Y (multiclass), kind 3 = max(0, (1-Y)*Z + Y*(1-Z)) (bidirectional
 * hinge). reference: deepity/std/loss.py:131-151,162-163 */
int dbk_loss_terms(dbk_stream_t stream, int dtype, int kind, const void* Z, const void* Y, void* L, size_t n);
/* dZ = (Z - Y) * scale. reference: deepity/std/loss.py:98-112 */
int dbk_sub_scale(dbk_stream_t stream, int dtype, const void* Z, const void* Y, double scale, void* dZ, size_t n);
/* Gradient of the hinge loss: dZ = (1 - 2Y) * scale where (1-Y)*Z + Y*(1-Z) > 0, else 0.
 * reference: hinge._calc_dZ, deepity/std/loss.py:165-169 (dZ = 1-2Y, then maskout(L > 0, dZ)) */
int dbk_hinge_grad(dbk_stream_t stream, int dtype, const void* Z, const void* Y, double scale, void* dZ, size_t n);

/* The scan filters' constraint, applied to W (4m, nfilter) in place after every parameter update:
 * kind 0 ("pfm"): the four letter weights of every (tap, filter) become log(exp(w) / sum of the four exp(w));
 * kind 1 ("psam"): log(exp(w) / max of the four exp(w)); kind 2: w clipped to [lo, hi].
 * reference: corr1ord.enforce_constraints, kangaroo/kangaroo/_ext/corr1ord.py:60-77, called by the trainer
 * before the first and after every step (deepity/deepity/sgd.py:103-107,137). */
int dbk_corr1ord_constraint(dbk_stream_t stream, int dtype, void* W, size_t m, size_t nfilter, int kind, double lo, double hi);

/* ------------------------------------------------------------------ fused dense head for scoring */

/* scores[r, b] = head_b(pooled[r, b*k:(b+1)*k]) for nblock models with k inputs each:
 * hidden > 0: relu(x.W1_b + b1_b).W2_b + b2_b ; hidden == 0: x.W1_b + b1_b ; then logistic if
 * apply_logistic. W1 (k*nblock, hidden|1), b1 (1, hidden*nblock | nblock), W2 (hidden*nblock, 1), b2 (1, nblock).
 * in_scale multiplies the inputs (test-time dropout rescale, one value per model, may be NULL).
 * nfeat > 0: every model's block of W1 has k + nfeat rows, the last nfeat of them weighting the columns of
 * feats (n, nfeat), a feature matrix shared by all models and not scaled by in_scale (the reference's
 * combiner input X1, kangaroo/kangaroo/model.py:101-112); feats == NULL stands for all zeros, which is what
 * the reference's data source supplies (kangaroo/kangaroo/data.py:59-69).
 * Replaces blockwise_dot_combined -> bias -> relu -> blockwise_dot -> bias (-> logistic)
 * (reference: deepity/std/full.py:78-83,154-160, softmax.py:58-61). float32 only. */
int dbk_head_fprop(dbk_stream_t stream, size_t n, int nblock, int k, int hidden,
                   const float* pooled, int nfeat, const float* feats, const float* in_scale,
                   const float* W1, const float* b1, const float* W2, const float* b2,
                   int apply_logistic, float* scores);

/* Forward AND backward of the dense head for nblock models in two launches (workgroups of one model x
 * 32 rows, then an ordered sum over the row chunks):
 * dropout (rate per model, NULL = none; uniforms from U when given, else from the generator at
 * (seed, offset), or at (seed, *counter) when counter is a device pointer; after the masks are drawn
 * *counter is advanced by counter_advance) -> dense (+bias, ReLU, dense
 * when hidden > 0) -> bias -> logistic (loss_kind 0) or identity (loss_kind 1, 2) -> dA = (Z-Y)/n (loss_kind 2,
 * the hinge loss: (1-2Y)/n where (1-Y)Z + Y(1-Z) > 0, else 0) masked by
 * Ymask (may be NULL) and, with reverse_complement, by the pair rule of dbk_calc_zmask -> all gradients.
 * Writes Z (n, nblock), dpooled (n, k*nblock), dW1, db1, dW2, db2 (overwritten, not accumulated) and,
 * if loss is not NULL, the per-model mean loss (nblock). Masks drawn here equal those of
 * dbk_dropout_fp_tr for the same (seed, offset). float32. Deterministic.
 * nfeat, feats: shared feature columns as in dbk_head_fprop (no dropout on them, no gradient back to them;
 * W1 and dW1 then have k + nfeat rows per model).
 * Replaces the reference's layer-by-layer head in a training step (deepity/std/elemwise.py:71-180,
 * full.py:78-119, softmax.py:58-77, loss.py:98-119,157-174). */
int dbk_head_train(dbk_stream_t stream, size_t n, int nblock, int k, int hidden, int loss_kind, int reverse_complement,
                   const float* pooled, int nfeat, const float* feats, const float* rate, const float* U, uint64_t seed, uint64_t offset,
                   uint64_t* counter, uint64_t counter_advance,
                   const float* W1, const float* b1, const float* W2, const float* b2,
                   const float* Y, const uint8_t* Ymask,
                   float* Z, float* dpooled, float* dW1, float* db1, float* dW2, float* db2, float* loss);
/* counter[0] += delta on the device (advances a generator position kept in device memory, so that a
 * captured HIP graph draws fresh masks on every replay). */
int dbk_counter_add(dbk_stream_t stream, uint64_t* counter, uint64_t delta);

/* ------------------------------------------------------------------ one whole optimiser step */

/* Everything one step of a group of `nmodel` same-architecture models touches. The parameters, their
 * gradients and the momentum live in flat float32 vectors of nparam elements, as the reference trainer
 * keeps them (deepity/deepity/sgd.py:287-331); off_* are the element offsets of the blocks inside them:
 * Wc (4m, nmodel*nfilter), bc (nmodel*nfilter), W1 (k*nmodel, hidden|1), b1 (hidden*nmodel | nmodel),
 * W2 (hidden*nmodel, 1), b2 (nmodel) with k = nfilter (x2 for all-pooling); W2 / b2 only when hidden > 0.
 * Work buffers are the caller's: pooled and dpooled (nregion, k*nmodel), argmax (nregion,
 * nmodel*nfilter; unused for avg pooling), Z (nregion, nmodel), and with input dropout Xdrop, Mdrop (N). */
typedef struct dbk_train_step_args {
    size_t nmodel, nfilter, m, hidden;      /* architecture: filters per model, filter length, hidden units (0 = none) */
    int ptype, loss_kind;                   /* DBK_PT_MAX / AVG / ALL; 0 = logistic + nll, 1 = identity + mse, 2 = identity + hinge */
    int reverse_complement, nesterov;
    size_t nparam;
    float *P, *dP, *mP;
    const float *drate, *mrate;             /* per-element learning and momentum rates */
    size_t off_Wc, off_bc, off_W1, off_b1, off_W2, off_b2;
    const uint8_t* X; size_t N;             /* packed batch (see dbk_corr1ord) */
    const uint32_t* regions; size_t nregion; /* (nregion, 2) row ranges */
    const float* Y; const uint8_t* Ymask;   /* targets (nregion, nmodel); mask may be NULL */
    float input_rate;                       /* input-base dropout rate, 0 = off */
    uint8_t *Xdrop, *Mdrop;
    const float* rate;                      /* pooled-feature dropout rate per model, NULL = off */
    uint64_t seed; uint64_t* counter;       /* generator seed and its position in device memory */
    const float* decay;                     /* L1 coefficient per element of P, NULL while decay is off */
    int freeze_scan;                        /* zero the scan filters' gradient (filters not yet training) */
    float* pooled; uint32_t* argmax; float* Z; float* dpooled;
    float* loss;                            /* per-model mean loss (nmodel), may be NULL */
    uint64_t* act;                          /* activity masks (see dbk_scanpool_fprop), N * ceil(nmodel*nfilter/64) words; may be NULL */
    float* L;                               /* look-ahead vector (nparam), may be NULL: see dbk_gradstep_lookahead */
    int L_ready;                            /* L already holds P + mrate*mP (left there by the previous step) */
    size_t nfeat; const float* feats;       /* shared feature columns (nregion, nfeat) entering the first dense layer after each model's
                                               pooled features: W1 is ((k+nfeat)*nmodel, hidden|1); feats NULL = all zeros
                                               (reference: kangaroo/kangaroo/model.py:101-112, data.py:59-69) */
} dbk_train_step_args;

/* One optimiser step, all launches issued from native code on `stream`:
 * [Nesterov look-ahead] -> [input dropout] -> dbk_scanpool_fprop -> dbk_head_train -> dbk_scanpool_bprop
 * -> [dbk_l1_decay] -> [zero dWc] -> momentum / Nesterov update. Bit-identical to calling those entry
 * points one by one; exists because a step on a small minibatch is bound by the host's cost per launch.
 * With a look-ahead vector L (Nesterov only) the step reads its weights from L and ends by writing the
 * next step's look-ahead there, so consecutive steps need no launch for it (L_ready).
 * reference: the body of the trainer's loop, deepity/deepity/sgd.py:98-135 (gradstep with the batch
 * gradient as callback, deepity_smat.py:77-117, gradstep.cu:41-72). */
int dbk_train_step(dbk_stream_t stream, const dbk_train_step_args* args);
/* One step of each of `ngroup` model groups that train on the same batch (same N, regions, nregion and filter
 * length; architectures may differ: pooling type, hidden units, models per group), e.g. the architectures of
 * one calibration batch. Every phase of the step is one launch that holds the grids of all the groups, so
 * groups that are each too small to fill the GPU run side by side on one stream, with no second stream and
 * no event. Each group's results are the bits its own dbk_train_step gives. Up to 8 groups, each with a
 * look-ahead vector (Nesterov) and filters of at most 24 taps, are taken together; any other call steps
 * the groups one after the other on `stream`.
 * reference: the per-architecture loop over one shared minibatch in the calibration search, which trains
 * all sampled models on the same batches (deepity/deepity/hpsearch.py:314-330, sgd.py:98-135). */
int dbk_train_steps(dbk_stream_t stream, size_t ngroup, const dbk_train_step_args* const* args);
/* The same step for a SMALL group in ONE launch: 1-4 models with at most 64 filters (of at most 32 taps) between
 * them, Nesterov momentum, no input dropout, at most 4096 regions of at most 256 rows each. A workgroup takes one
 * region (up to 256 regions; a few beyond) through forward, dense head and backward without leaving the CU, and after
 * one grid-wide barrier (bounded wait) all workgroups add up their shares of the gradient in a fixed order and apply
 * the update. With reverse-complement pairs and one region per workgroup, the two workgroups of a pair show each other
 * their predictions through the workspace (bounded wait, status 1 if it runs out).
 * Reads pooled / argmax / dpooled / act / L of the block not at all (weights come from P + mrate * mP); writes Z,
 * dP, mP, P, loss and advances the generator position. Deterministic; within the tolerances of dbk_train_step,
 * not its bits (other summation orders).
 * work: caller-owned device memory of dbk_train_step_single_workspace() bytes, 16-byte aligned, ZERO before its
 * first use and from then on passed unchanged to every call with the same nregion. Word 0 (uint32) counts the
 * launches that stepped; word 1 is a status: 1 = a workgroup waited too long (at the barrier or for its
 * reverse-complement partner), 2 = a region had more than 256 rows. Whether a launch steps is decided once for the
 * whole grid (a compare-and-swap on one word of the workspace): an abandoned launch changes no parameter, neither
 * momentum nor generator position, and sets the status; while the status is non-zero every further launch on that
 * workspace returns without doing anything. To go on, wait for the stream, read words 0 and 1, and zero the first
 * 32768 bytes of the workspace (status alone is not enough: the barrier's words hold the abandoned launch's number).
 * Calls that share a workspace must not overlap. *work_bytes = 0 from the query means the shape is not taken
 * (use dbk_train_step).
 * reference: the body of the trainer's loop, deepity/deepity/sgd.py:98-135, as dbk_train_step. */
int dbk_train_step_single_workspace(const dbk_train_step_args* args, size_t* work_bytes);
int dbk_train_step_single(dbk_stream_t stream, const dbk_train_step_args* args, void* work, size_t work_bytes);
/* sizeof(dbk_train_step_args) as the library was built, for bindings that mirror the block field by field. */
int dbk_train_step_args_size(void);

#ifdef __cplusplus
}
#endif
#endif /* DEEPBIND_HIP_H */
