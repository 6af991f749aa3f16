// XLA FFI handlers over the C ABI of libgla_hip.so: the binding behind which a JAX-ROCm build of
// zhixuan-lin/gla-jax would reach the gfx950 kernels.  The reference has no FFI of its own; its boundary is
// the pair of jax.custom_vjp rules of chunk_gla (gla.py:628-655) and recurrent_gla (gla.py:362-388, 441), and
// the two scan operators of ops.py (ops.py:234-284, 396-456).  One handler per rule; every handler is an
// argument adapter and nothing else: shapes are read off the buffers, the stream comes from XLA, the status
// code of the C entry point becomes an ffi::Error.
//
// STATUS: source only.  It needs xla/ffi/api/ffi.h (shipped inside jaxlib: `python -c "import jaxlib,
// os; print(os.path.join(os.path.dirname(jaxlib.__file__), 'include'))"`), which the machines this library
// was built and tested on do not have, so this file has never been compiled; gla_jax_amd/build.py compiles
// it only when that header is found.
//
// Array layout.  The reference's functions are unbatched ([T,H,D], hidden [H,DK,DV]) and batched with
// jax.vmap (gla.py:1335).  The handlers are registered with vmap_method="broadcast_all" on the Python
// side, so every mapped axis arrives as a leading dimension of EVERY operand; all leading dimensions are
// folded into the batch argument of the C ABI.
#include <cstdint>
#include <string>

#include "xla/ffi/api/ffi.h"

#include "gla_hip.h"

namespace ffi = xla::ffi;

namespace {

struct Dims {
    int64_t B = 1, T = 0, H = 0, DK = 0, DV = 0;
    bool ok = false;
};

// key is [..., T, H, DK], value is [..., T, H, DV]; everything in front of T is batch.
Dims dims_of(const ffi::AnyBuffer &key, const ffi::AnyBuffer &value)
{
    Dims d;
    auto kd = key.dimensions(), vd = value.dimensions();
    if (kd.size() < 3 || vd.size() != kd.size()) return d;
    const size_t n = kd.size();
    for (size_t i = 0; i + 3 < n; ++i) {
        if (kd[i] != vd[i]) return d;
        d.B *= kd[i];
    }
    d.T = kd[n - 3];
    d.H = kd[n - 2];
    d.DK = kd[n - 1];
    d.DV = vd[n - 1];
    d.ok = vd[n - 3] == d.T && vd[n - 2] == d.H;
    return d;
}

bool dtype_of(ffi::DataType t, gla_dtype *out)
{
    if (t == ffi::DataType::BF16) { *out = GLA_BF16; return true; }
    if (t == ffi::DataType::F32) { *out = GLA_F32; return true; }
    return false;
}

ffi::Error status(const char *fn, int rc)
{
    if (rc == 0) return ffi::Error::Success();
    if (rc < 0) return ffi::Error::InvalidArgument(std::string(fn) + ": " + gla_status_string(rc));
    return ffi::Error::Internal(std::string(fn) + ": " + gla_status_string(rc));
}

// ---- chunk_gla ---------------------------------------------------------------------------------------------
// forward rule, chunk_gla_forward (gla.py:483-550).  Results: hidden_final, out, the residual `states`
// (the analogue of the saved `state`, gla.py:548) and a workspace XLA allocates for the call; the Python side
// sizes the last two with gla_chunk_states_bytes / gla_chunk_fwd_workspace_bytes.
ffi::Error ChunkFwd(hipStream_t stream, int64_t chunk_size, ffi::AnyBuffer h0, ffi::Buffer<ffi::F32> g,
                    ffi::AnyBuffer v, ffi::AnyBuffer k, ffi::AnyBuffer q, ffi::Result<ffi::AnyBuffer> hT,
                    ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> states,
                    ffi::Result<ffi::AnyBuffer> workspace)
{
    Dims d = dims_of(k, v);
    gla_dtype dt, hdt;                       // the state arrays carry a dtype of their own (gla.py:711-716, 727)
    if (!d.ok || !dtype_of(v.element_type(), &dt) || !dtype_of(h0.element_type(), &hdt) ||
        hT->element_type() != h0.element_type())
        return ffi::Error::InvalidArgument("gla_chunk_fwd: bad operands");
    return status("gla_chunk_fwd",
                  gla_chunk_fwd(stream, d.B, d.T, d.H, d.DK, d.DV, chunk_size, dt, hdt, h0.untyped_data(),
                                g.typed_data(), v.untyped_data(), k.untyped_data(), q.untyped_data(),
                                hT->untyped_data(), out->untyped_data(), states->untyped_data(),
                                workspace->untyped_data(), workspace->size_bytes()));
}

// backward rule, chunk_gla_backward (gla.py:552-625): cotangents in, gradients out in argument order
// (hidden_init, log_fgate, value, key, query; gla.py:625).
ffi::Error ChunkBwd(hipStream_t stream, int64_t chunk_size, ffi::Buffer<ffi::F32> g, ffi::AnyBuffer v,
                    ffi::AnyBuffer k, ffi::AnyBuffer q, ffi::AnyBuffer states, ffi::AnyBuffer dhT,
                    ffi::AnyBuffer dout, ffi::Result<ffi::AnyBuffer> dh0, ffi::Result<ffi::Buffer<ffi::F32>> dg,
                    ffi::Result<ffi::AnyBuffer> dv, ffi::Result<ffi::AnyBuffer> dk,
                    ffi::Result<ffi::AnyBuffer> dq, ffi::Result<ffi::AnyBuffer> workspace)
{
    Dims d = dims_of(k, v);
    gla_dtype dt, hdt;
    if (!d.ok || !dtype_of(v.element_type(), &dt) || !dtype_of(dhT.element_type(), &hdt) ||
        dh0->element_type() != dhT.element_type())
        return ffi::Error::InvalidArgument("gla_chunk_bwd: bad operands");
    return status("gla_chunk_bwd",
                  gla_chunk_bwd(stream, d.B, d.T, d.H, d.DK, d.DV, chunk_size, dt, hdt, g.typed_data(),
                                v.untyped_data(), k.untyped_data(), q.untyped_data(), states.untyped_data(),
                                dhT.untyped_data(), dout.untyped_data(), dh0->untyped_data(), dg->typed_data(),
                                dv->untyped_data(), dk->untyped_data(), dq->untyped_data(),
                                workspace->untyped_data(), workspace->size_bytes()));
}

// ---- recurrent_gla -----------------------------------------------------------------------------------------
// forward rule, recurrent_gla_forward (gla.py:99-170); `reverse` as in gla.py:421-438.  The element type of
// `out` selects the flavour: the value dtype for recurrent_gla, F32 for recurrent_gla_naive (gla.py:37).  The last
// result is a workspace XLA allocates for the call, sized by gla_recurrent_fwd_workspace_bytes on the Python side
// (head dimension 256 and calls with few long sequences use one; elsewhere it is a few bytes that nobody reads).
ffi::Error RecurrentFwd(hipStream_t stream, bool reverse, ffi::AnyBuffer h0, ffi::Buffer<ffi::F32> g,
                        ffi::AnyBuffer v, ffi::AnyBuffer k, ffi::AnyBuffer q, ffi::Result<ffi::AnyBuffer> hT,
                        ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::AnyBuffer> workspace)
{
    Dims d = dims_of(k, v);
    gla_dtype dt, hdt, odt;
    if (!d.ok || !dtype_of(v.element_type(), &dt) || !dtype_of(out->element_type(), &odt) ||
        !dtype_of(h0.element_type(), &hdt) || hT->element_type() != h0.element_type())
        return ffi::Error::InvalidArgument("gla_recurrent_fwd: bad operands");
    return status("gla_recurrent_fwd_ws",
                  gla_recurrent_fwd_ws(stream, d.B, d.T, d.H, d.DK, d.DV, dt, hdt, odt, reverse ? 1 : 0,
                                       h0.untyped_data(), g.typed_data(), v.untyped_data(), k.untyped_data(),
                                       q.untyped_data(), hT->untyped_data(), out->untyped_data(),
                                       workspace->untyped_data(), workspace->size_bytes()));
}

// backward rule, recurrent_gla_backward (gla.py:172-269); residuals (h0, g, v, k, q, hidden_final), gla.py:169.
ffi::Error RecurrentBwd(hipStream_t stream, bool reverse, ffi::AnyBuffer h0, ffi::Buffer<ffi::F32> g,
                        ffi::AnyBuffer v, ffi::AnyBuffer k, ffi::AnyBuffer q, ffi::AnyBuffer hT,
                        ffi::AnyBuffer dhT, ffi::AnyBuffer dout, ffi::Result<ffi::AnyBuffer> dh0,
                        ffi::Result<ffi::Buffer<ffi::F32>> dg, ffi::Result<ffi::AnyBuffer> dv,
                        ffi::Result<ffi::AnyBuffer> dk, ffi::Result<ffi::AnyBuffer> dq,
                        ffi::Result<ffi::AnyBuffer> workspace)
{
    Dims d = dims_of(k, v);
    gla_dtype dt, hdt, odt;
    if (!d.ok || !dtype_of(v.element_type(), &dt) || !dtype_of(dout.element_type(), &odt) ||
        !dtype_of(h0.element_type(), &hdt) || hT.element_type() != h0.element_type() ||
        dhT.element_type() != h0.element_type() || dh0->element_type() != h0.element_type())
        return ffi::Error::InvalidArgument("gla_recurrent_bwd: bad operands");
    return status("gla_recurrent_bwd_ws",
                  gla_recurrent_bwd_ws(stream, d.B, d.T, d.H, d.DK, d.DV, dt, hdt, odt, reverse ? 1 : 0,
                                       h0.untyped_data(), g.typed_data(), v.untyped_data(), k.untyped_data(),
                                       q.untyped_data(), hT.untyped_data(), dhT.untyped_data(), dout.untyped_data(),
                                       dh0->untyped_data(), dg->typed_data(), dv->untyped_data(),
                                       dk->untyped_data(), dq->untyped_data(), workspace->untyped_data(),
                                       workspace->size_bytes()));
}

// ---- the scans of ops.py -----------------------------------------------------------------------------------
// cumsum_recursive(src, axis, init, reverse) (ops.py:234-284).  The Python side moves nothing: it passes the
// scanned axis as an attribute and the handler views src as [n_outer, t_len, n_inner].  `init` has the shape
// of src without the scanned axis; an absent init is passed as an array of zeros.
ffi::Error Cumsum(hipStream_t stream, int64_t axis, bool reverse, ffi::Buffer<ffi::F32> src,
                  ffi::Buffer<ffi::F32> init, ffi::Result<ffi::Buffer<ffi::F32>> dst)
{
    auto sd = src.dimensions();
    const int64_t n = (int64_t)sd.size();
    if (axis < 0) axis += n;
    if (axis < 0 || axis >= n) return ffi::Error::InvalidArgument("gla_cumsum_f32: axis out of range");
    int64_t outer = 1, inner = 1;
    for (int64_t i = 0; i < axis; ++i) outer *= sd[i];
    for (int64_t i = axis + 1; i < n; ++i) inner *= sd[i];
    return status("gla_cumsum_f32", gla_cumsum_f32(stream, src.typed_data(), init.typed_data(), dst->typed_data(),
                                                   outer, sd[axis], inner, reverse ? 1 : 0));
}

// rnn_recursive(log_fgate[T,K], kv[T,K,V], init_log_fgate[K], init_kv[K,V], reverse) (ops.py:396-456);
// leading dimensions in front of T are independent problems.
ffi::Error RnnScan(hipStream_t stream, bool reverse, ffi::Buffer<ffi::F32> log_fgate, ffi::Buffer<ffi::F32> kv,
                   ffi::Buffer<ffi::F32> init_log_fgate, ffi::Buffer<ffi::F32> init_kv,
                   ffi::Result<ffi::Buffer<ffi::F32>> out_log_lambda, ffi::Result<ffi::Buffer<ffi::F32>> out_state)
{
    auto kd = kv.dimensions();
    if (kd.size() < 3) return ffi::Error::InvalidArgument("gla_rnn_scan_f32: kv must be [..., T, K, V]");
    const size_t n = kd.size();
    int64_t batch = 1;
    for (size_t i = 0; i + 3 < n; ++i) batch *= kd[i];
    return status("gla_rnn_scan_f32",
                  gla_rnn_scan_f32(stream, log_fgate.typed_data(), kv.typed_data(), init_log_fgate.typed_data(),
                                   init_kv.typed_data(), out_log_lambda->typed_data(), out_state->typed_data(),
                                   batch, kd[n - 3], kd[n - 2], kd[n - 1], reverse ? 1 : 0));
}

}  // namespace

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaChunkFwd, ChunkFwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<int64_t>("chunk_size")
                                  .Arg<ffi::AnyBuffer>()          // hidden_init
                                  .Arg<ffi::Buffer<ffi::F32>>()   // log_fgate
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::AnyBuffer>()          // key
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Ret<ffi::AnyBuffer>()          // hidden_final
                                  .Ret<ffi::AnyBuffer>()          // out
                                  .Ret<ffi::AnyBuffer>()          // states (residual)
                                  .Ret<ffi::AnyBuffer>());        // workspace

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaChunkBwd, ChunkBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<int64_t>("chunk_size")
                                  .Arg<ffi::Buffer<ffi::F32>>()   // log_fgate
                                  .Arg<ffi::AnyBuffer>()          // value
                                  .Arg<ffi::AnyBuffer>()          // key
                                  .Arg<ffi::AnyBuffer>()          // query
                                  .Arg<ffi::AnyBuffer>()          // states
                                  .Arg<ffi::AnyBuffer>()          // dhidden_final
                                  .Arg<ffi::AnyBuffer>()          // dout
                                  .Ret<ffi::AnyBuffer>()          // dhidden_init
                                  .Ret<ffi::Buffer<ffi::F32>>()   // dlog_fgate
                                  .Ret<ffi::AnyBuffer>()          // dvalue
                                  .Ret<ffi::AnyBuffer>()          // dkey
                                  .Ret<ffi::AnyBuffer>()          // dquery
                                  .Ret<ffi::AnyBuffer>());        // workspace

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaRecurrentFwd, RecurrentFwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<bool>("reverse")
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>());        // workspace

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaRecurrentBwd, RecurrentBwd,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<bool>("reverse")
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()
                                  .Arg<ffi::AnyBuffer>()          // hidden_final
                                  .Arg<ffi::AnyBuffer>()          // dhidden_final
                                  .Arg<ffi::AnyBuffer>()          // dout
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>()
                                  .Ret<ffi::AnyBuffer>());        // workspace

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaCumsum, Cumsum,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<int64_t>("axis")
                                  .Attr<bool>("reverse")
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(GlaRnnScan, RnnScan,
                              ffi::Ffi::Bind()
                                  .Ctx<ffi::PlatformStream<hipStream_t>>()
                                  .Attr<bool>("reverse")
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Arg<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>()
                                  .Ret<ffi::Buffer<ffi::F32>>());
