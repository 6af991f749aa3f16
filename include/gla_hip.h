/* gla_hip.h — C ABI of libgla_hip.so: the MI355X (gfx950) kernels behind the Gated Linear Attention
 * hot path of zhixuan-lin/gla-jax.
 *
 * The reference has no FFI of its own: its boundary is the Python call signature of chunk_gla /
 * recurrent_gla plus their jax.custom_vjp rules (gla.py:657-692, 628-655; gla.py:405-441,
 * 362-388).  Each entry point below replaces one forward or backward rule of that boundary, for a
 * whole batch at once (the reference batches with jax.vmap, gla.py:1335; here B is an argument).
 *
 * Conventions, all entry points:
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it, nothing synchronises.
 *   - All pointers are device pointers, 16-byte aligned, dense row-major:
 *       log_fgate/key/query  [B, T, H, DK]     value/out/dout  [B, T, H, DV]
 *       hidden_*             [B, H, DK, DV]
 *     log_fgate and its gradient are always float32 (gla.py:495 intent); `dtype` is the element
 *     type of value/key/query and of every output that mirrors them (out.dtype == value.dtype,
 *     gla.py:538); `hidden_dtype` is the element type of the four state arrays hidden_init,
 *     hidden_final, dhidden_final and dhidden_init, whatever `dtype` is: the reference loads
 *     hidden_init in its own dtype into an fp32 state and stores hidden_final back in it
 *     (gla.py:44-46, 89-97, 727), and hands it uncast to the chunk scan (gla.py:711-716), so an
 *     fp32 state carried from one segment of a sequence to the next next to bf16 value/key/query
 *     is not rounded at the hand-over.
 *   - The library never allocates, frees or synchronises: outputs and workspaces are the caller's.
 *   - Return value: 0 = enqueued; < 0 = argument rejected on the host before any launch (see
 *     gla_status); > 0 = a hipError_t from a launch.  No C++ exception crosses the boundary.
 *   - Re-entrant.  The only state kept between calls is set-up that is done once per device and never
 *     changes afterwards: the grant of more than 64 KB of LDS to the kernels that need it, and the device
 *     address of the static scratch array of gla_chunk_fwd_static.
 */
#ifndef GLA_HIP_H_
#define GLA_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define GLA_HIP_ABI_VERSION 3

typedef enum gla_dtype {
    GLA_F32 = 0,
    GLA_BF16 = 1
} gla_dtype;

typedef enum gla_status {
    GLA_OK = 0,
    GLA_ERR_NULL = -1,         /* a required pointer is NULL */
    GLA_ERR_SHAPE = -2,        /* a dimension is <= 0 or not a supported multiple */
    GLA_ERR_DTYPE = -3,        /* unknown dtype enum */
    GLA_ERR_CHUNK = -4,        /* chunk_size not a supported power of two or does not divide T
                                  (the reference asserts both: gla.py:500, einops gla.py:674) */
    GLA_ERR_WORKSPACE = -5,    /* workspace too small / NULL */
    GLA_ERR_ALIGN = -6,        /* pointer not 16-byte aligned */
    GLA_ERR_UNSUPPORTED = -7   /* valid in the reference but not built here (see message) */
} gla_status;

/* Library identification.  No reference counterpart. */
int gla_abi_version(void);
/* Static, thread-safe description of a status code returned by any entry point. */
const char *gla_status_string(int status);

/* ---- scans (ops.py) -------------------------------------------------------------------------- */

/* Replaces cumsum_recursive(src, axis, init, reverse) (ops.py:234-284; kernel ops.py:152-162).
 * src/dst are viewed as [n_outer, t_len, n_inner] float32, the scan runs along t_len in fp32;
 * init is [n_outer, n_inner] or NULL (zero).  reverse != 0 sums from the far end.  dst must not alias src. */
int gla_cumsum_f32(void *stream, const float *src, const float *init, float *dst,
                   int64_t n_outer, int64_t t_len, int64_t n_inner, int reverse);

/* Replaces rnn_recursive(log_fgate[T,K], kv[T,K,V], init_log_fgate[K], init_kv[K,V], reverse)
 * (ops.py:396-456; kernel ops.py:299-334; combine op ops.py:286-297), for `batch` independent
 * problems laid out back to back:
 *   forward: x_n = exp(a_n)[:,None]*x_{n-1} + b_n, x_{-1} = init_kv ; reverse: x_n = exp(a_n)*x_{n+1} + b_n.
 * out_log_lambda [T,K] receives the running sum of a (including init_log_fgate), out_state [T,K,V]
 * the states.  init pointers may be NULL (zeros); out_log_lambda may be NULL.  All float32.  Any V >= 1:
 * a multiple of 4 moves 16 bytes per access (kv, init_kv and out_state then 16-byte aligned), other V
 * one float. */
int gla_rnn_scan_f32(void *stream, const float *log_fgate, const float *kv,
                     const float *init_log_fgate, const float *init_kv,
                     float *out_log_lambda, float *out_state,
                     int64_t batch, int64_t T, int64_t K, int64_t V, int reverse);

/* ---- recurrent_gla (gla.py:405-441) ---------------------------------------------------------- */

/* Replaces recurrent_gla_forward (gla.py:99-170, kernel gla.py:50-96): the per-timestep recurrence
 * S_t = exp(g_t)*S_{t-1} + k_t v_t^T, o_t = S_t^T q_t with the state in fp32 registers; no hidden
 * state is written except hidden_final.  reverse != 0 scans t = T-1..0 with outputs left in place
 * (gla.py:421-438).  out_dtype is the element type of `out` (value dtype for recurrent_gla,
 * GLA_F32 for the recurrent_gla_naive flavour whose output is fp32 by promotion, gla.py:37).
 * Requires DK == DV (gla.py:120) in {16, 32, 64, 128, 256}. */
int gla_recurrent_fwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                      gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                      const void *hidden_init, const float *log_fgate, const void *value,
                      const void *key, const void *query,
                      void *hidden_final, void *out);

/* Replaces recurrent_gla_backward (gla.py:172-269, kernel gla.py:271-360): sweep 1 recomputes S_t
 * and forms dq_t; sweep 2 runs backwards for dk_t, dv_t and d(hidden_init); d(log_fgate) is the
 * reverse cumsum identity of gla.py:263 accumulated in fp32 inside sweep 2.  `hidden_final` is the
 * forward's residual (gla.py:169); it is checked but not read: the term sum_v dhidden_final * hidden_final
 * of gla.py:263 is formed from the fp32 state sweep 1 ends with, not from its stored rounding.
 * dlog_fgate doubles as the fp32 scratch that carries q*dq from sweep 1 to sweep 2, so no workspace is
 * needed.  dout has element type out_dtype. */
int gla_recurrent_bwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                      gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                      const void *hidden_init, const float *log_fgate, const void *value,
                      const void *key, const void *query, const void *hidden_final,
                      const void *dhidden_final, const void *dout,
                      void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery);

/* The same two rules (gla.py:99-170, 172-269) with a caller-provided workspace, which buys two things.
 * (1) At head dimension 256 the recurrence runs as four problems of head dimension 128 (it is a sum over key
 * features and independent over value features): two passes of the 128-feature kernels over 2H heads, on the
 * matrix cores for bf16 data, with the passes' results kept in fp32 in the workspace and rounded once.  Without a
 * workspace (the two entry points above) head dimension 256 runs on per-timestep vector kernels, an order of
 * magnitude slower.
 * (2) With few sequences (B*H, at head dimension 256 2*B*H, at most half of the GPU's 256 compute units for bf16
 * data at head dimensions 64 and more, a quarter otherwise) and T a multiple of S segments of at least 128 steps
 * (64 at head dimensions 128 and 256 while few workgroups result), every sequence runs as S segments side by side:
 * the recurrence is linear in the state, so one pass from zero states gives each segment's own contribution, a scan
 * over the segments the state that enters each (fp32, in the workspace), and a second pass the outputs; the
 * backward does the same for the states' cotangents first.  One workgroup walks one (batch, head) pair, so without
 * this a call with 8 pairs uses 8 of 256 compute units.  The backward uses its result arrays as scratch until it
 * writes the results there (where the first passes are full kernels: the gates moved by one row in dlog_fgate, the
 * passes' unused `out` in dquery and dkey); an fp32 dout beside bf16 data (out_dtype != dtype) enters the cotangents' pass as two bf16 arrays, head and
 * remainder, kept in dkey and dvalue (head dimensions 16 and 32 then run the backward on whole sequences).
 * The size functions return 0 where a workspace buys nothing; the entry points then ignore `workspace` (NULL is
 * fine) and behave exactly like the ones above.  Same results within the tolerance either way (segments: the
 * same but for the order of fp32 sums). */
size_t gla_recurrent_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype);
size_t gla_recurrent_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV, gla_dtype dtype);
int gla_recurrent_fwd_ws(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                         const void *hidden_init, const float *log_fgate, const void *value,
                         const void *key, const void *query,
                         void *hidden_final, void *out, void *workspace, size_t workspace_bytes);
int gla_recurrent_bwd_ws(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         gla_dtype dtype, gla_dtype hidden_dtype, gla_dtype out_dtype, int reverse,
                         const void *hidden_init, const float *log_fgate, const void *value,
                         const void *key, const void *query, const void *hidden_final,
                         const void *dhidden_final, const void *dout,
                         void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery,
                         void *workspace, size_t workspace_bytes);

/* ---- chunk_gla (gla.py:657-692) -------------------------------------------------------------- */

/* Bytes of the `states` residual written by gla_chunk_fwd and read by gla_chunk_bwd: the
 * states before every chunk and after the last one, [B,H,T/C+1,DK,DV] in the element type, the analogue of
 * the reference's saved `state` (gla.py:548, 729; its last slice is hidden_final, gla.py:720-723).  C is
 * the tile the kernels run with: the largest one built that divides T (the result does not depend on the
 * chunk length, so chunk_size is validated and otherwise not used).  The layout inside is the library's own (a
 * 16-bit state lies as 32 x 32 tiles; at head dimension 256 there are two such arrays for [B,2H] heads of 128
 * features, one per pass of the 128-feature kernels).  Returns 0 for unsupported arguments. */
size_t gla_chunk_states_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                              int64_t chunk_size, gla_dtype dtype);
/* Bytes of scratch needed by gla_chunk_fwd / gla_chunk_bwd (DK == DV in {16, 32, 64, 128, 256}).  Returns 0 for
 * unsupported arguments. */
size_t gla_chunk_fwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                     int64_t chunk_size, gla_dtype dtype);
size_t gla_chunk_bwd_workspace_bytes(int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                                     int64_t chunk_size, gla_dtype dtype);

/* Replaces chunk_gla_forward (gla.py:483-550) and everything under it: the log-gate cumsum
 * (ops.py:234), compute_intra_contrib (gla.py:792-855) with compute_score (gla.py:964-1029),
 * compute_inter_contrib (gla.py:695-729) and the chunk state scan (ops.py:396).  Requires
 * DK == DV (gla.py:499), T % chunk_size == 0, chunk_size a power of two >= 32.  `states` receives the
 * residual for the backward; pass NULL when no gradient will be taken.  hidden_init enters the fp32 scan
 * in hidden_dtype (gla.py:711-716); only its copy as the first chunk's incoming state is stored in `dtype`
 * like every other chunk state (gla.py:719-720). */
int gla_chunk_fwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                  int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                  const void *hidden_init, const float *log_fgate, const void *value,
                  const void *key, const void *query,
                  void *hidden_final, void *out, void *states,
                  void *workspace, size_t workspace_bytes);

/* Replaces chunk_gla_backward (gla.py:552-625) and everything under it
 * (compute_intra_contrib_backward gla.py:857-960, compute_score backward gla.py:1036-1189,
 * compute_inter_contrib_backward gla.py:731-790, the reverse state scan and the reverse cumsum
 * gla.py:616-617).  Gradients come back in argument order (gla.py:625). */
int gla_chunk_bwd(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                  int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                  const float *log_fgate, const void *value, const void *key, const void *query,
                  const void *states, const void *dhidden_final, const void *dout,
                  void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery,
                  void *workspace, size_t workspace_bytes);

/* gla_chunk_fwd for callers that cannot allocate device memory and have no workspace to pass: code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments and results as gla_chunk_fwd without the workspace pair: the per-chunk products,
 * decays and chunk-start states go through a static device array of GLA_CHUNK_FWD_STATIC_BYTES bytes
 * (80 MiB: the headline shape B4 T4096 H6 D128 bf16 needs 49.1 MiB) that every GPU the library runs on holds
 * from the first call on it until the process ends.  Shapes whose workspace (gla_chunk_fwd_workspace_bytes)
 * exceeds the capacity are rejected with GLA_ERR_WORKSPACE before anything is launched.  The call allocates
 * and frees nothing.  The first call on a device looks up the array's address there (hipGetSymbolAddress):
 * make it outside a graph capture.  All calls on one GPU share the one array: calls that overlap in time on
 * the same GPU (different streams, different host threads) race and must be serialised by the caller; calls
 * in order on one stream are safe, nothing in the array has to survive from one call to the next. */
#define GLA_CHUNK_FWD_STATIC_BYTES ((size_t)80 << 20)
int gla_chunk_fwd_static(void *stream, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                         const void *hidden_init, const float *log_fgate, const void *value,
                         const void *key, const void *query,
                         void *hidden_final, void *out, void *states);

/* Same as gla_chunk_fwd / gla_chunk_bwd but launching only the kernels selected by `stages`
 * (bit 0: per-chunk outer products, bit 1: scan over chunks, bit 2: output / gradient kernel), the
 * others' results being taken from the workspace and residual buffers of an earlier full call with
 * the same arguments.  No counterpart in the reference; exists so that a caller can time one kernel
 * with events on its own stream (bench.py does). */
int gla_chunk_fwd_stages(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                         const void *hidden_init, const float *log_fgate, const void *value,
                         const void *key, const void *query,
                         void *hidden_final, void *out, void *states,
                         void *workspace, size_t workspace_bytes);
int gla_chunk_bwd_stages(void *stream, int stages, int64_t B, int64_t T, int64_t H, int64_t DK, int64_t DV,
                         int64_t chunk_size, gla_dtype dtype, gla_dtype hidden_dtype,
                         const float *log_fgate, const void *value, const void *key, const void *query,
                         const void *states, const void *dhidden_final, const void *dout,
                         void *dhidden_init, float *dlog_fgate, void *dvalue, void *dkey, void *dquery,
                         void *workspace, size_t workspace_bytes);

#ifdef __cplusplus
}
#endif
#endif /* GLA_HIP_H_ */
