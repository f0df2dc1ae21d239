/*
 * hpx — MI355X (gfx950) gradient-compression kernels behind a plain C ABI.
 *
 * This is the drop-in boundary for the reference extension's kernel-driver
 * layer: each entry point below replaces one of the nine `hp_cuda_*` free
 * functions the reference declares in hp_cuda.cpp:18-102 and defines in
 * hp_cuda_kernel.cu.  The reference passes std::vector<T*>/std::vector<int32_t>
 * argument lists and a cudaStream_t; here the same lists arrive as `count`
 * plus parallel arrays of plain pointers and sizes, and the stream as an opaque
 * hipStream_t.  Argument order and meaning follow the reference function named
 * in each comment.
 *
 * Conventions
 *   - All tensor pointers are DEVICE pointers into caller-owned memory; the
 *     pointer/size arrays themselves are HOST arrays read during the call.
 *   - Calls enqueue work on `stream` and return without waiting, except where a
 *     comment says otherwise.  The reference's drivers print and continue on a
 *     body failure; these entry points return the code instead:
 *       0   success
 *      -1   the reference body's own failure (bad bitwidth, short message)
 *      -2   a HIP runtime error (hpx_last_error() has the text)
 *      -3   an argument the kernels cannot take (null pointer, negative size)
 *   - The library owns a small grow-only device workspace per (device, stream).
 *     Entry points may be called from several host threads; calls that share a
 *     stream are serialised while they enqueue.
 *   - Sizes are int32 element/byte counts exactly as in the reference.
 *   - Tuning options: see hpx_set_option.
 */
#ifndef HPX_H_
#define HPX_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* hpx_stream_t; /* a hipStream_t; NULL is the null stream */

#define HPX_OK 0
#define HPX_ERR_BODY (-1)
#define HPX_ERR_HIP (-2)
#define HPX_ERR_ARG (-3)

/* Library version (major*10000 + minor*100 + patch). */
int hpx_version(void);
/* Text of the last failure on the calling thread ("" if none). */
const char* hpx_last_error(void);
/* Releases every workspace the library allocated (all devices, all streams).
 * No call may be in flight.  No counterpart in the reference (its scratch is
 * the caller's output buffer). */
int hpx_release_workspaces(void);
/* Waits for `stream`, then frees the workspace the library keeps for (current
 * device, stream) and hands back the stream's claim on the grid-barrier kernels
 * (see hpx_terngrad_encode), so that another stream can take it.  Call it before
 * destroying a stream on which codecs ran; no other call may use the stream at
 * the same time.  A stream that is used again afterwards simply gets a new
 * workspace.  No counterpart in the reference. */
int hpx_release_stream(hpx_stream_t stream);

/* ---- tuning options -------------------------------------------------------
 * No counterpart in the reference.  An option starts from the environment
 * variable HPX_<NAME IN CAPITALS> when that is set, else from its default, and
 * can be changed at any time (it applies to calls made afterwards):
 *   "stream_store_max_bytes"  total output size up to which the write-only
 *                             decoders use streaming stores (default: no
 *                             limit; lower it if the next kernel reads the
 *                             decoded tensor straight back)
 *   "terngrad_resident_min"   smallest tensor, in elements, that
 *                             hpx_terngrad_encode sends through its
 *                             single-launch resident kernel (default 5 * 2^20,
 *                             where it starts to beat the two-launch encode;
 *                             negative: never)
 *   "terngrad_barrier_ms"     bound on that kernel's grid-barrier wait
 *                             (default 2000)
 *   "terngrad_resident_bucket" 1 (default): a call with 2 to 192 tensors of one
 *                             bit width and rounding mode that add up to at
 *                             least terngrad_resident_min elements and fit the
 *                             chip together takes ONE resident launch for all of
 *                             them; 0: each tensor is looked at on its own
 *   "terngrad_resident_workgroups" workgroups of a resident launch; 0
 *                             (default): one per CU of the device.  A process
 *                             that may only use some of the CUs (a CU mask)
 *                             must set it to that number: the workgroups of a
 *                             resident launch wait for each other
 *   "terngrad_resident_streamed" 1 (default): a tensor larger than the chip
 *                             holds (about 33.5 M elements) also takes ONE
 *                             launch of that kind: its head stays on chip,
 *                             the rest is read twice by the same launch;
 *                             0: such tensors take the two-launch encode
 *   "gd_provisional_min_samples" a sparsifier call (hpx_gd_encode,
 *                             hpx_dgc_encode) whose tensors' samples add up to
 *                             at least this many (default -1: none) starts its
 *                             pass over the tensors from a provisional
 *                             threshold taken from the first 16384 samples and
 *                             finds the exact one afterwards among the samples
 *                             the pass marked, instead of gathering the whole
 *                             sample first; the message is the same.  Negative:
 *                             never.  Off by default: measured on a 138 M
 *                             element tensor it is 3 % slower than the gather
 *   "gd_provisional_margin"   how many times the expected number of entries
 *                             the provisional threshold lets through (default
 *                             3).  A tensor whose provisional threshold turns
 *                             out not to lie below the exact one is encoded
 *                             again through the gather path (hpx_gd_fallbacks
 *                             counts them); 0 all but forces that
 *   "clock_seed"              what an encoder uses when it is called with
 *                             seeds == NULL; negative (default): the wall
 *                             clock, as the reference's bodies
 *                             (terngrad_body.h:247-251, gd_body.h:138-140).
 *                             Lets the C++ drivers, whose signatures carry no
 *                             seed, produce reproducible messages
 * Unknown names return HPX_ERR_ARG. */
int hpx_set_option(const char* name, int64_t value);
int hpx_get_option(const char* name, int64_t* value);

/* ---- measurement aid ------------------------------------------------------
 * No counterpart in the reference.  While enabled, every kernel the library
 * launches carries a pair of HIP events that take the kernel's own begin and
 * end times on the stream of the launch (hipExtLaunchKernelGGL), so the
 * durations are those a kernel trace shows, without the hand-over between
 * launches; hpx_profile_query waits for them and returns the summed duration
 * and the number of launches of the kernel with that name (e.g.
 * "terngrad_decode_kernel").  hpx_profile_reset forgets what was recorded.
 * Off by default; leave it off while a stream is being captured into a graph
 * (a launch with events is not something a graph can record). */
int hpx_profile_enable(int on);
int hpx_profile_reset(void);
int hpx_profile_query(const char* kernel, double* total_ms, int64_t* launches);

/* ---- TBQ: threshold quantisation with residual feedback ------------------ */

/* Replaces hp_cuda_tbq (hp_cuda.cpp:52-61, hp_cuda_kernel.cu:120-158; body
 * tbq_body.h:90-158).  For tensor t: residual += grad; each element becomes a
 * 2-bit code (1: |r|<thr, 2: r>=thr then r-=thr, 0: r<=-thr then r+=thr), four
 * codes per byte LSB-first, unused fields of the last byte stay 1.
 * outs[t] needs (sizes[t]+3)/4 bytes.  grads are read-only.  The reference's
 * unused size arguments (residual sizes, out sizes) are not part of this ABI.
 * All tensors go out in one launch sequence; no host synchronisation (the
 * reference's trailing cudaStreamSynchronize is left to the caller). */
int hpx_tbq_encode(int count, const float* const* grads, const int32_t* sizes,
                   float* const* residuals, uint8_t* const* outs,
                   const float* thresholds, hpx_stream_t stream);

/* Replaces hp_cuda_tbqr (hp_cuda.cpp:41-50, hp_cuda_kernel.cu:161-198; body
 * tbq_body.h:160-200).  outs[t][i] = (code-1)*thr, added to the existing value
 * when is_add_tos[t] != 0.  The same output may be named by several messages
 * (the reference's root path decodes every gathered message into one tensor,
 * hp_cuda.cpp:241-259): they are applied in call order, and when the outputs are
 * exact duplicates all messages of a tensor are applied in a single pass over
 * it with the same sequence of fp32 additions.  (When the messages of each
 * tensor lie at one distance from each other - the slots of a gathered buffer,
 * with or without the one slot a root leaves out - a call with up to 208
 * tensors is a single launch.) */
int hpx_tbq_decode(int count, float* const* outs, const int32_t* sizes,
                   const uint8_t* const* ins, const float* thresholds,
                   const int32_t* is_add_tos, hpx_stream_t stream);

/* ---- TernGrad: b-bit min/max quantiser, b in {1,2,4,8} -------------------- */

/* Replaces hp_cuda_terngrad (hp_cuda.cpp:21-29, hp_cuda_kernel.cu:30-65; body
 * terngrad_body.h:162-307).  Message layout: [0]=bitwidth, [1]=unused slots in
 * the last byte, [2:6]=min, [6:10]=max (fp32 LE), [10:] codes LSB-first.
 * out_sizes[t] must be 10 + ceil(n/(8/b)): a partial last byte is written at
 * outs[t][out_sizes[t]-1] as in the reference (and always rounds to nearest).
 * enable_randoms[t] != 0 selects stochastic rounding with the reference's LCG
 * seeded per output byte from seeds[t] + byte index.  The reference takes that
 * seed from the wall clock inside the body (terngrad_body.h:247-251); pass
 * seeds == NULL for that behaviour, or an array of `count` values to fix it.
 * Returns -1 without launching if any bitwidth is not 1, 2, 4 or 8
 * (terngrad_body.h:207-212).
 * A tensor between "terngrad_resident_min" and about 33M elements (16M at
 * 1 bit) is encoded by one launch that keeps it in registers and LDS between the
 * min/max pass and the quantise pass, with a grid-wide barrier in between.  That
 * barrier needs every CU of the device to be reachable from `stream` (no CU
 * mask), and two such kernels must never run at once, so per device only the
 * first stream that encodes a large tensor uses this kernel (other streams keep
 * to the two-launch path; hpx_release_stream hands the claim back).  The wait is
 * bounded: if it ever expires (the GPU is shared with another process's barrier
 * kernels, say) that launch leaves its message unwritten.  The library keeps a
 * record of every tensor such a launch encoded; hpx_terngrad_encode_status
 * (below) waits for the stream and, if a barrier expired, encodes those tensors
 * again through the two-launch path, with the seeds they were given, so the
 * message that should have come out does.  A later hpx_terngrad_encode on the
 * stream that finds the expiry does the same before its own work, without
 * waiting.  Either way the stream keeps to the two-launch path from then on.
 * The reference's driver returns with a valid message (it synchronises,
 * hp_cuda_kernel.cu:30-65): a caller that reads a message on the host, or hands
 * it on, calls hpx_terngrad_encode_status first, and leaves the inputs
 * untouched until then.
 * Not recordable into a HIP graph (per-call tags travel in the kernel
 * arguments): returns -3 on a stream that is being captured.
 * A call with several tensors is first cut into groups of consecutive tensors
 * of one bit width and rounding mode (at most 192) that fit the chip together;
 * a group of two or more that adds up to "terngrad_resident_min" elements is
 * encoded by one launch of the same kind (option "terngrad_resident_bucket",
 * same conditions on `stream`); what is left over goes tensor by tensor as
 * described above.  The bytes written do not depend on the route. */
int hpx_terngrad_encode(int count, const float* const* ins, const int32_t* in_sizes,
                        uint8_t* const* outs, const int32_t* out_sizes,
                        const uint8_t* bitwidths, const int32_t* enable_randoms,
                        const uint64_t* seeds, hpx_stream_t stream);

/* One half of the completion contract of hp_cuda_terngrad (hp_cuda_kernel.cu:30-65
 * returns only once terngrad_body has synchronised after its last quantise
 * launch, terngrad_body.h:285, so every message is complete and the reference's
 * scheduler reads it on another stream at once, hp_cuda.cpp:464-468).  This call
 * settles the launches that meet at a grid barrier, the only ones that can leave
 * a message unwritten: it returns 0 at once if none is outstanding on `stream`
 * - it does NOT wait for two-launch encodes, which cannot fail but may still be
 * queued or running; a caller that needs them finished waits for the stream
 * itself, as the C++ driver hp_cuda_terngrad (csrc/hp_cuda_shim.cpp) does after
 * this call.  Otherwise it waits for the stream; if a barrier wait expired, it
 * encodes the tensors of those launches again through the two-launch path on
 * the same stream and waits for that too.  On return 0 no message of any
 * hpx_terngrad_encode call made on the stream so far will be left unwritten;
 * -2 if the repair itself failed.  hpx_terngrad_repaired counts the tensors
 * ever encoded again on the stream (a diagnostic). */
int hpx_terngrad_encode_status(hpx_stream_t stream);
int64_t hpx_terngrad_repaired(hpx_stream_t stream);

/* Measurement aid, no counterpart in the reference.  While a device buffer of
 * 4 * workgroups 64-bit words is set, every workgroup b of a single-launch
 * (resident) encode leaves four readings of the GPU's 100 MHz wall clock in
 * words 4b .. 4b+3: on entry, before its first load is requested; when its
 * whole share is loaded and reduced; when it has the global extremes (the
 * grid-wide exchange is behind it); when its last store has been issued.
 * bench.py turns them into the per-phase breakdown of the headline kernel.
 * Launches with more workgroups than the buffer holds leave nothing.  NULL or
 * 0 switches it off (the default); the caller keeps the buffer alive until
 * then and until the launches that saw it have finished. */
int hpx_terngrad_phase_stamps(uint64_t* device_words, int32_t workgroups);

/* hpx_terngrad_encode for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference.  Same arguments, same bytes out; always the two-launch path
 * (min/max, then quantise), whose reduction slots live in a fixed device array
 * of 576 KiB inside the library instead of a workspace, so the call makes no
 * hipMalloc / hipFree, takes no workspace, never waits for the stream and puts
 * no per-call tag into its kernels (it clears the slots it uses with a small
 * kernel first), which also makes it recordable into a graph (seeds == NULL then
 * freezes the clock value of the capture: every replay rounds with the same
 * draws).  The first call on a device looks up the array's address
 * (hipGetDevice, hipGetSymbolAddress), which a capture in a non-relaxed mode
 * does not allow: make one eager call per device - any size - before capturing.
 * Limits: at most 192 tensors per call
 * (-3 beyond that).  Every call on a GPU shares that GPU's array: calls that
 * overlap in time on one GPU - on any streams - race; order them. */
int hpx_terngrad_encode_noalloc(int count, const float* const* ins, const int32_t* in_sizes,
                                uint8_t* const* outs, const int32_t* out_sizes,
                                const uint8_t* bitwidths, const int32_t* enable_randoms,
                                const uint64_t* seeds, hpx_stream_t stream);

/* Replaces hp_cuda_terngradr (hp_cuda.cpp:31-38, hp_cuda_kernel.cu:200-230;
 * body terngrad_body.h:309-409).  The header is parsed on the device, so the
 * call does not wait for the stream (the reference copies it to the host and
 * synchronises).  The element count is ((in_size-10)*(8/b)) - tail as in the
 * reference, and is additionally clamped to out_sizes[t] so a malformed header
 * cannot write outside the output.  A message whose bitwidth byte is invalid
 * decodes to nothing and raises the sticky flag hpx_terngrad_decode_status
 * reports.  Several messages may name the same output (hp_cuda.cpp:421-439);
 * they are applied in call order, in a single pass over the tensor when the
 * outputs are exact duplicates (and a call with up to 208 tensors whose
 * messages lie at one distance from each other is a single launch, as for
 * hpx_tbq_decode). */
int hpx_terngrad_decode(int count, float* const* outs, const int32_t* out_sizes,
                        const uint8_t* const* ins, const int32_t* in_sizes,
                        const int32_t* is_add_tos, hpx_stream_t stream);

/* Waits for `stream`, then returns -1 if any hpx_terngrad_decode on it since
 * the last status call met an invalid bitwidth byte (the reference's
 * terngrad_r_body failure, terngrad_body.h:352-355), else 0. */
int hpx_terngrad_decode_status(hpx_stream_t stream);

/* ---- GradDrop ("DGC"): sampled-threshold top-k sparsifier ----------------- */

/* Replaces hp_cuda_gd (hp_cuda.cpp:64-73, hp_cuda_kernel.cu:67-94; body
 * gd_body.h:102-232).  Per tensor: residual += grad; threshold = the
 * int(sample_cnt*(1-drop))-th largest of sample_cnt = ceil(N*sample_rate)
 * sampled |residual| values (indices from the reference's LCG seeded with
 * seeds[t] + sample number); select {i : r[i] > thr || r[i] < -thr}; if more
 * than ceil(N*(1-drop)) were selected keep that many largest |r|.  Message:
 * int32 4+8k, k int32 indices, k fp32 values; residual[idx] = 0.  Indices are
 * ascending when nothing was cut and in descending |r| order when cut (ties:
 * ascending index).  seeds == NULL takes the wall clock (gd_body.h:138-140).
 * Unlike the reference, bytes of outs[t] past the message are left untouched
 * (scratch lives in the library workspace), so outs[t] needs only
 * 4 + 8*ceil(N*(1-drop)) bytes.
 * All tensors of a call go through each phase together (one launch per phase
 * for up to 256 tensors), so hand over whole buckets, as the reference's
 * scheduler does (hp_cuda.cpp:284-301).  The reference waits for the stream
 * three times per tensor; this call never waits for the stream: it polls
 * pinned host words in which a kernel reports the candidate count of every
 * tensor (while later kernels are still running), queues the sort-and-cut for
 * the tensors that overshoot and returns; results are stream-ordered.  Because
 * of that dependence on the host it returns -3 on a stream that is being
 * captured into a graph; so do hpx_gd_decode and the two DGC calls.
 * A tensor whose parameters make no sense (threshold index outside the sample)
 * is skipped and makes the call return -3; the other tensors are encoded, as
 * the reference driver prints and goes on (hp_cuda_kernel.cu:90-92). */
int hpx_gd_encode(int count, const float* const* grads, const int32_t* Ns,
                  float* const* residuals, uint8_t* const* outs,
                  const double* sample_rates, const double* drop_ratios,
                  const uint64_t* seeds, hpx_stream_t stream);

/* Replaces hp_cuda_gdr (hp_cuda.cpp:75-82, hp_cuda_kernel.cu:96-118; body
 * gd_body.h:283-353).  Reads every header first (one wait on the stream, as in
 * the reference); returns -1 before touching any output if a message is longer
 * than its in_sizes[t].  is_add_tos[t] == 0 zero-fills out_sizes[t] elements
 * and then scatters; otherwise accumulates. */
int hpx_gd_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes,
                  float* const* outs, const int32_t* out_sizes,
                  const int32_t* is_add_tos, hpx_stream_t stream);

/* Diagnostic: tensors of sparsifier calls on `stream` so far whose provisional
 * threshold was not below the exact one and that were therefore encoded through
 * the gather path after all (see "gd_provisional_margin"). */
int64_t hpx_gd_fallbacks(hpx_stream_t stream);

/* ---- DGC without residual --------------------------------------------------
 * The reference holds this sparsifier as a body without a driver
 * (dgc_with_auxiliary_body / dgc_body, dgc_body.h:71-152 / :155-226; dgc_r_body
 * :252-293); these two entry points are the drivers it would have.
 * Encode is hpx_gd_encode with the gradient in the place of the residual:
 * nothing is added, the threshold is the int(sample_cnt*s_percent)-th largest of
 * sample_cnt = ceil(N*sample_rate) sampled |G|, entries beyond it (at most
 * ceil(N*s_percent), the largest first if there are more) go into the message
 * and are CLEARED IN grads[t].  Same message layout, same output size
 * 4 + 8*ceil(N*s_percent), same way of learning the counts.
 * Decode differs from hpx_gd_decode in write mode only: the output is not
 * cleared first (dgc_body.h:283-289). */
int hpx_dgc_encode(int count, float* const* grads, const int32_t* Ns, uint8_t* const* outs,
                   const double* sample_rates, const double* s_percents,
                   const uint64_t* seeds, hpx_stream_t stream);
int hpx_dgc_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes,
                   float* const* outs, const int32_t* out_sizes,
                   const int32_t* is_add_tos, hpx_stream_t stream);

/* ---- ECQ: error-compensated quantiser with a history -----------------------
 * The reference holds this codec as a body without a driver or a caller
 * (ecq_body / ecq_r_body, ecq_body.h:157-286 / :342-423); these two entry points
 * are the drivers it would have.  The body keeps its |G + alpha*H| scratch at the
 * start of the output buffer and writes the packed bytes over it, which is only
 * well defined under its serial policy; that serial behaviour is what is
 * reproduced, bit for bit, quirks included:
 *   message  [0:4] int32 10 + M, [4:8] max|G + alpha*H| (fp32), [8] bitwidth,
 *            [9] unused slots of the last byte, [10:] M = ceil(N/(8/b)) bytes of
 *            b-bit codes LSB-first, code = uint8((|G + alpha*H| + max) / gap + u),
 *            gap = max / (2^(b-1) - 1), u from the reference's LCG seeded with
 *            seeds[t] + byte index (NULL: the wall clock, ecq_body.h:253-255);
 *   history  H = beta*H + (unrounded - code) * gap;
 *   quirks   the quantise loop covers M - 1 bytes: the LAST payload byte is not a
 *            code byte (it holds one byte of the scratch, or stays as the caller
 *            left it when N <= 2) and the history of its elements is not updated;
 *            for 4- and 8-bit codes scratch elements 2 (and 3) are read after a
 *            payload byte has been stored into them; codes come out of an absolute
 *            value, so decoded values are >= 0 (the sign is lost); max < 1e-6
 *            gives zero bytes and H *= beta.
 * outs[t] needs 10 + M bytes (the reference needs 4*N for its scratch).
 * bitwidths must be 2, 4 or 8 (-1 otherwise; the reference aborts).
 * Encode only enqueues work; decode reads every header first (one wait on the
 * stream, as the reference copies the header to the host) and returns -1 if an
 * output is smaller than its message's element count (the reference aborts).
 * out[x] = code*gap - max, added to the existing value when is_add_tos[t] != 0. */
int hpx_ecq_encode(int count, const float* const* Gs, const int32_t* Ns, float* const* Hs, uint8_t* const* outs,
                   const int32_t* out_sizes, const double* alphas, const double* betas, const int32_t* bitwidths,
                   const uint64_t* seeds, hpx_stream_t stream);
int hpx_ecq_decode(int count, const uint8_t* const* ins, const int32_t* in_sizes, float* const* outs,
                   const int32_t* out_sizes, const int32_t* is_add_tos, hpx_stream_t stream);

/* ---- PowerSGD: rank-r factorisation with error feedback ------------------- */
/* The reference bodies operate on torch tensors (powersgd_body.h); here every
 * matrix is a row-major fp32 device array: M is n x m, Q is m x r, P is n x r,
 * grad/residual hold numel <= n*m elements (the flat prefix of M).  Any rank
 * r >= 1, as the reference (its bodies are plain mm, powersgd_body.h:28,49,69):
 * up to 16 in one pass over the matrix, above that sixteen columns of the
 * factors per pass. */

/* Replaces hp_cuda_powersgd_encode1 (hp_cuda.cpp:85-92,
 * hp_cuda_kernel.cu:232-255; powersgd_body.h:10-31 as its comments state it):
 * M.flat[:numel] = grad + residual;  P = M * Q. */
int hpx_powersgd_encode1(int count, const float* const* grads, const int64_t* numels,
                         const float* const* residuals, const float* const* Qs,
                         float* const* Ms, float* const* Ps, const int32_t* ns,
                         const int32_t* ms, const int32_t* rs, hpx_stream_t stream);

/* Replaces hp_cuda_powersgd_encode2 (hp_cuda.cpp:93-98,
 * hp_cuda_kernel.cu:257-276; powersgd_body.h:33-52): P <- orthonormal basis of
 * its columns (modified Gram-Schmidt; equals the reference's Householder Q
 * factor up to the sign of each column), then Q = M^T * P. */
int hpx_powersgd_encode2(int count, float* const* Ps, const float* const* Ms,
                         float* const* Qs, const int32_t* ns, const int32_t* ms,
                         const int32_t* rs, hpx_stream_t stream);

/* Replaces hp_cuda_powersgd_decode (hp_cuda.cpp:99-106,
 * hp_cuda_kernel.cu:278-301; powersgd_body.h:54-78): M = P * Q^T;
 * residual = grad - M.flat[:numel];  grad = M.flat[:numel]. */
int hpx_powersgd_decode(int count, const float* const* Ps, const float* const* Qs,
                        float* const* Ms, float* const* residuals, float* const* grads,
                        const int64_t* numels, const int32_t* ns, const int32_t* ms,
                        const int32_t* rs, hpx_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* HPX_H_ */
