// torch.ops.catccos.*: the operator-library face of the HIP library, as a C++ translation unit.
//
// Mirrors the reference's torch binding (examples/torch_binding/src/torch_bindings.cpp:84-239:
// `TORCH_LIBRARY(catccos, m)` with `init` / `<op>` / `finalize`, state in a function-local static, inputs
// checked with TORCH_CHECK and made contiguous, output allocated here, current stream taken, the extern "C"
// wrapper called; the device implementation registered for the accelerator key only) and its Meta twin
// (examples/torch_binding/src/torch_bindings_meta.cpp:18-35: output shapes only), for the compute halves
// this library holds instead of `allgather_matmul`.  There is no communication here, so `init` accepts
// rank_size == 1 only and makes no use of local_mem_size / ip_port (the symmetric heap they size is the
// part that was dropped).
//
// Behaviour kept from the reference: an operator called before `init` fails with the reference's message
// (torch_bindings.cpp:131-133); `init` checks its arguments like the reference and is a no-op the second
// time (:88-95); `finalize` on an uninitialised library returns 0 (:205-207).
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <algorithm>
#include <atomic>
#include <cctype>
#include <initializer_list>
#include <mutex>
#include <string>
#include <tuple>

#include "catccos_hip.h"

namespace {

struct CatccosTorchState {
    std::atomic<bool> initialized{false};   // read without the lock by every operator
    std::atomic<bool> launched{false};      // some operator of this library has put work on a stream
    int64_t rank_id = -1, rank_size = 0;
    std::mutex mu;
};

CatccosTorchState &State()
{
    static CatccosTorchState state;
    return state;
}

void NeedInit()
{
    TORCH_CHECK(State().initialized.load(std::memory_order_acquire), "catccos TORCH_LIBRARY not initialized, call torch.ops.catccos.init(...) first");
}

// Every tensor argument of a device kernel must live on the GPU of the first one.  The dispatcher picks the GPU
// kernel as soon as one argument is a GPU tensor; a host tensor among the others (group sizes often live on the
// host) would hand a host address to a kernel (the reference checks the same, torch_bindings.cpp:140-144).  Called
// before anything is allocated or launched.
struct NamedTensor {
    const char *name;
    const at::Tensor &t;
};
void SameDevice(const char *op, std::initializer_list<NamedTensor> args)
{
    const NamedTensor &first = *args.begin();
    for (const NamedTensor &a : args) {
        TORCH_CHECK(a.t.defined(), "catccos::", op, ": ", a.name, " is undefined");
        TORCH_CHECK(a.t.is_cuda(), "catccos::", op, ": ", a.name, " must be a GPU tensor, got one on ", a.t.device());
        TORCH_CHECK(a.t.device() == first.t.device(), "catccos::", op, ": ", a.name, " is on ", a.t.device(), " but ", first.name, " is on ",
                    first.t.device());
    }
}

int FormatCode(const std::string &name)
{
    std::string s = name;
    std::transform(s.begin(), s.end(), s.begin(), [](unsigned char c) { return std::tolower(c); });
    if (s == "e4m3" || s == "fp8") return CCH_FMT_E4M3;
    if (s == "e5m2") return CCH_FMT_E5M2;
    if (s == "e2m1" || s == "fp4") return CCH_FMT_E2M1;
    if (s == "e1m2") return CCH_FMT_E1M2;
    TORCH_CHECK(false, "unknown MX payload format '", name, "'");
    return -1;
}

bool IsFp4(int fmt) { return fmt == CCH_FMT_E2M1 || fmt == CCH_FMT_E1M2; }
int64_t ScaleCols(int64_t k) { return 2 * ((k + 63) / 64); }   // E8M0 bytes per row: block count padded to even

// (a ROCm build of PyTorch presents its HIP devices and streams under the names of the GPU key: the stream of a
// tensor's device is asked for through that front)
void *StreamOf(const at::Tensor &t)
{
    State().launched.store(true, std::memory_order_release);
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

void Check(int rc, const char *what) { TORCH_CHECK(rc == CCH_OK, "catccos::", what, ": ", cch_last_error()); }

at::Tensor Bytes(const at::Tensor &like, at::IntArrayRef shape) { return at::empty(shape, like.options().dtype(at::kByte)); }

// ---------------------------------------------------------------------------------------------
// init / finalize (reference torch_bindings.cpp:85-121, :203-229)

int64_t Init(int64_t rank_id, int64_t rank_size, int64_t local_mem_size, std::string ip_port)
{
    auto &st = State();
    std::lock_guard<std::mutex> lock(st.mu);
    if (st.initialized.load()) return 0;
    TORCH_CHECK(rank_id >= 0, "invalid rank_id: ", rank_id);
    TORCH_CHECK(rank_size > 0, "invalid rank_size: ", rank_size);
    TORCH_CHECK(local_mem_size > 0, "invalid local_mem_size: ", local_mem_size);
    TORCH_CHECK(!ip_port.empty(), "ip_port is empty");
    TORCH_CHECK(rank_size == 1 && rank_id == 0, "catccos on one GPU has no peers: rank_size must be 1 and rank_id 0, got ", rank_id, " of ",
                rank_size);
    st.rank_id = rank_id;
    st.rank_size = rank_size;
    st.initialized.store(true, std::memory_order_release);
    return 0;
}

int64_t Finalize()
{
    auto &st = State();
    std::lock_guard<std::mutex> lock(st.mu);
    if (!st.initialized.load()) return 0;
    // the reference drains its stream before it lets go of its buffers; a process in which no operator of this
    // library ever launched (only init / finalize or Meta-shape calls) has nothing to drain and must not create a
    // GPU context here
    if (st.launched.load(std::memory_order_acquire)) (void)hipStreamSynchronize(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
    st.initialized.store(false, std::memory_order_release);
    st.rank_id = -1;
    st.rank_size = 0;
    return 0;
}

// ---------------------------------------------------------------------------------------------
// shape helpers shared by the device and the Meta kernels

struct MxShape {
    int fmt;
    int64_t t, n, k, e;
};

// a [T, K(/2)] payload with sa [T, ScaleCols(K)]; b [(E,) K, N(/2)] or [(E,) N, K(/2)] with sb of E * ScaleCols(K) * N bytes
MxShape MxShapes(const at::Tensor &a, const at::Tensor &sa, const at::Tensor &b, const at::Tensor &sb, const std::string &fmt_name, int64_t trans_b,
                 bool grouped)
{
    MxShape s;
    s.fmt = FormatCode(fmt_name);
    TORCH_CHECK(s.fmt != CCH_FMT_E1M2, "E1M2 is a quantiser format only: the matrix instructions have no such operand type");
    const int64_t pack = s.fmt == CCH_FMT_E2M1 ? 2 : 1;
    TORCH_CHECK(a.dim() == 2 && a.scalar_type() == at::kByte, "a must be a 2-D uint8 tensor");
    TORCH_CHECK(sa.dim() == 2 && sa.scalar_type() == at::kByte, "sa must be a 2-D uint8 tensor");
    TORCH_CHECK(b.dim() == (grouped ? 3 : 2) && b.scalar_type() == at::kByte && sb.scalar_type() == at::kByte, "b / sb must be uint8 tensors of rank ",
                grouped ? 3 : 2);
    s.t = a.size(0);
    s.k = a.size(1) * pack;
    const int64_t d0 = b.size(grouped ? 1 : 0), d1 = b.size(grouped ? 2 : 1);
    const int64_t kb = trans_b ? d1 * pack : d0;
    s.n = trans_b ? d0 : d1 * pack;
    TORCH_CHECK(kb == s.k, "inner dimensions differ: a gives K=", s.k, ", b gives K=", kb);
    TORCH_CHECK(sa.size(0) == s.t && sa.size(1) == ScaleCols(s.k), "sa must be [", s.t, ",", ScaleCols(s.k), "]");
    s.e = grouped ? b.size(0) : 1;
    TORCH_CHECK(sb.numel() == s.e * ScaleCols(s.k) * s.n, "sb has ", sb.numel(), " entries, expected ", s.e * ScaleCols(s.k) * s.n);
    return s;
}

void CheckGroups(const at::Tensor &group_sizes, int64_t e)
{
    TORCH_CHECK(group_sizes.dim() == 1 && group_sizes.scalar_type() == at::kInt, "group_sizes must be a 1-D int32 tensor");
    TORCH_CHECK(group_sizes.numel() == e, "group_sizes must have one entry per expert");
}

struct I8Shape {
    int64_t t, n, k, e;
};

I8Shape I8GroupedShapes(const at::Tensor &x, const at::Tensor &w, const at::Tensor &group_sizes, const at::Tensor &per_tok, const at::Tensor &per_ch,
                        int64_t trans_b)
{
    TORCH_CHECK(x.dim() == 2 && x.scalar_type() == at::kChar, "x must be a 2-D int8 tensor");
    TORCH_CHECK(w.dim() == 3 && w.scalar_type() == at::kChar, "w must be a 3-D int8 tensor");
    I8Shape s{x.size(0), trans_b ? w.size(1) : w.size(2), x.size(1), w.size(0)};
    TORCH_CHECK((trans_b ? w.size(2) : w.size(1)) == s.k, "shape mismatch between x and w");
    CheckGroups(group_sizes, s.e);
    TORCH_CHECK(per_tok.numel() == s.t && per_ch.dim() == 2 && per_ch.size(0) == s.e && per_ch.size(1) == s.n, "per_tok must be [T] and per_ch [E,N]");
    return s;
}

// ---------------------------------------------------------------------------------------------
// device kernels (registered for the GPU key)

std::tuple<at::Tensor, at::Tensor> MxQuant(const at::Tensor &x_in, std::string fmt_name, int64_t rounding)
{
    NeedInit();
    const int fmt = FormatCode(fmt_name);
    TORCH_CHECK(x_in.dim() == 2 && (x_in.scalar_type() == at::kBFloat16 || x_in.scalar_type() == at::kHalf),
                "mx_quant expects a 2-D bfloat16 (or float16) tensor");
    SameDevice("mx_quant", {{"x", x_in}});
    c10::DeviceGuard guard(x_in.device());
    const at::Tensor x = x_in.contiguous();
    const int64_t m = x.size(0), k = x.size(1);
    at::Tensor payload = Bytes(x, {m, IsFp4(fmt) ? (k + 1) / 2 : k}), scales = Bytes(x, {m, ScaleCols(k)});
    const int rc = x.scalar_type() == at::kHalf
                       ? cch_mx_quant_rows_f16(x.data_ptr(), payload.data_ptr(), scales.data_ptr(), m, k, fmt, (int)rounding, StreamOf(x))
                       : cch_mx_quant_rows(x.data_ptr(), payload.data_ptr(), scales.data_ptr(), m, k, fmt, (int)rounding, StreamOf(x));
    Check(rc, "mx_quant");
    return {payload, scales};
}

at::Tensor W8A8MatmulDequant(const at::Tensor &a_in, const at::Tensor &b_in, const at::Tensor &per_tok_in, const at::Tensor &per_ch_in, int64_t trans_b)
{
    NeedInit();
    TORCH_CHECK(a_in.dim() == 2 && a_in.scalar_type() == at::kChar, "a must be a 2-D int8 tensor");
    TORCH_CHECK(b_in.dim() == 2 && b_in.scalar_type() == at::kChar, "b must be a 2-D int8 tensor");
    SameDevice("w8a8_matmul_dequant", {{"a", a_in}, {"b", b_in}, {"per_tok", per_tok_in}, {"per_ch", per_ch_in}});
    c10::DeviceGuard guard(a_in.device());
    const at::Tensor a = a_in.contiguous(), b = b_in.contiguous();
    const int64_t m = a.size(0), k = a.size(1), n = trans_b ? b.size(0) : b.size(1);
    TORCH_CHECK((trans_b ? b.size(1) : b.size(0)) == k, "inner dimensions differ");
    const at::Tensor per_tok = per_tok_in.contiguous().to(at::kFloat), per_ch = per_ch_in.contiguous().to(at::kFloat);
    TORCH_CHECK(per_tok.numel() == m && per_ch.numel() == n, "per_tok must have M entries and per_ch N entries");
    at::Tensor out = at::empty({m, n}, a.options().dtype(at::kBFloat16));
    Check(cch_gemm_i8_dequant_out(a.data_ptr(), b.data_ptr(), per_tok.data_ptr<float>(), per_ch.data_ptr<float>(), out.data_ptr(), m, n, k, (int)trans_b,
                                  CCH_OUT_BF16, StreamOf(a)),
          "w8a8_matmul_dequant");
    return out;
}

at::Tensor MxMatmul(const at::Tensor &a_in, const at::Tensor &sa_in, const at::Tensor &b_in, const at::Tensor &sb_in, std::string fmt_name, int64_t trans_b)
{
    NeedInit();
    SameDevice("mx_matmul", {{"a", a_in}, {"sa", sa_in}, {"b", b_in}, {"sb", sb_in}});
    c10::DeviceGuard guard(a_in.device());
    const at::Tensor a = a_in.contiguous(), sa = sa_in.contiguous(), b = b_in.contiguous(), sb = sb_in.contiguous();
    const MxShape s = MxShapes(a, sa, b, sb, fmt_name, trans_b, false);
    at::Tensor out = at::empty({s.t, s.n}, a.options().dtype(at::kBFloat16));
    Check(cch_mx_gemm_out(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), out.data_ptr(), s.t, s.n, s.k, s.fmt, (int)trans_b, CCH_OUT_BF16,
                          StreamOf(a)),
          "mx_matmul");
    return out;
}

at::Tensor GmmDequantSwiglu(const at::Tensor &x_in, const at::Tensor &w_in, const at::Tensor &gs_in, const at::Tensor &per_tok_in,
                            const at::Tensor &per_ch_in, int64_t trans_b)
{
    NeedInit();
    SameDevice("gmm_dequant_swiglu", {{"x", x_in}, {"w", w_in}, {"group_sizes", gs_in}, {"per_tok", per_tok_in}, {"per_ch", per_ch_in}});
    c10::DeviceGuard guard(x_in.device());
    const at::Tensor x = x_in.contiguous(), w = w_in.contiguous(), gs = gs_in.contiguous();
    const at::Tensor per_tok = per_tok_in.contiguous().to(at::kFloat), per_ch = per_ch_in.contiguous().to(at::kFloat);
    const I8Shape s = I8GroupedShapes(x, w, gs, per_tok, per_ch, trans_b);
    at::Tensor out = at::empty({s.t, s.n / 2}, x.options().dtype(at::kBFloat16));
    Check(cch_gmm_i8_dequant_swiglu_out(x.data_ptr(), w.data_ptr(), gs.data_ptr<int32_t>(), per_tok.data_ptr<float>(), per_ch.data_ptr<float>(),
                                        out.data_ptr(), s.e, s.t, s.n, s.k, (int)trans_b, CCH_OUT_BF16, StreamOf(x)),
          "gmm_dequant_swiglu");
    return out;
}

std::tuple<at::Tensor, at::Tensor> GmmDequantSwigluMx(const at::Tensor &x_in, const at::Tensor &w_in, const at::Tensor &gs_in, const at::Tensor &per_tok_in,
                                                      const at::Tensor &per_ch_in, int64_t trans_b, std::string fmt_name)
{
    NeedInit();
    const int fmt = FormatCode(fmt_name);
    SameDevice("gmm_dequant_swiglu_mx", {{"x", x_in}, {"w", w_in}, {"group_sizes", gs_in}, {"per_tok", per_tok_in}, {"per_ch", per_ch_in}});
    c10::DeviceGuard guard(x_in.device());
    const at::Tensor x = x_in.contiguous(), w = w_in.contiguous(), gs = gs_in.contiguous();
    const at::Tensor per_tok = per_tok_in.contiguous().to(at::kFloat), per_ch = per_ch_in.contiguous().to(at::kFloat);
    const I8Shape s = I8GroupedShapes(x, w, gs, per_tok, per_ch, trans_b);
    TORCH_CHECK(s.n % 2 == 0 && (fmt != CCH_FMT_E2M1 || s.n % 4 == 0), "n must be even (a multiple of 4 for FP4 output)");
    const int64_t h = s.n / 2;
    at::Tensor payload = Bytes(x, {s.t, fmt == CCH_FMT_E2M1 ? h / 2 : h}), scales = Bytes(x, {s.t, ScaleCols(h)});
    Check(cch_gmm_i8_dequant_swiglu_mx(x.data_ptr(), w.data_ptr(), gs.data_ptr<int32_t>(), per_tok.data_ptr<float>(), per_ch.data_ptr<float>(),
                                       payload.data_ptr(), scales.data_ptr(), s.e, s.t, s.n, s.k, (int)trans_b, fmt, StreamOf(x)),
          "gmm_dequant_swiglu_mx");
    return {payload, scales};
}

at::Tensor MxGroupedMatmul(const at::Tensor &a_in, const at::Tensor &sa_in, const at::Tensor &b_in, const at::Tensor &sb_in, const at::Tensor &gs_in,
                           std::string fmt_name, int64_t trans_b)
{
    NeedInit();
    SameDevice("mx_grouped_matmul", {{"a", a_in}, {"sa", sa_in}, {"b", b_in}, {"sb", sb_in}, {"group_sizes", gs_in}});
    c10::DeviceGuard guard(a_in.device());
    const at::Tensor a = a_in.contiguous(), sa = sa_in.contiguous(), b = b_in.contiguous(), sb = sb_in.contiguous(), gs = gs_in.contiguous();
    const MxShape s = MxShapes(a, sa, b, sb, fmt_name, trans_b, true);
    CheckGroups(gs, s.e);
    at::Tensor out = at::empty({s.t, s.n}, a.options().dtype(at::kBFloat16));
    Check(cch_mx_gmm(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), gs.data_ptr<int32_t>(), out.data_ptr(), s.e, s.t, s.n, s.k, s.fmt,
                     (int)trans_b, StreamOf(a)),
          "mx_grouped_matmul");
    return out;
}

std::tuple<at::Tensor, at::Tensor> MxGroupedMatmulSwigluMx(const at::Tensor &a_in, const at::Tensor &sa_in, const at::Tensor &b_in, const at::Tensor &sb_in,
                                                           const at::Tensor &gs_in, std::string fmt_name, int64_t trans_b, std::string out_fmt_name)
{
    NeedInit();
    const int ofmt = FormatCode(out_fmt_name);
    SameDevice("mx_grouped_matmul_swiglu_mx", {{"a", a_in}, {"sa", sa_in}, {"b", b_in}, {"sb", sb_in}, {"group_sizes", gs_in}});
    c10::DeviceGuard guard(a_in.device());
    const at::Tensor a = a_in.contiguous(), sa = sa_in.contiguous(), b = b_in.contiguous(), sb = sb_in.contiguous(), gs = gs_in.contiguous();
    const MxShape s = MxShapes(a, sa, b, sb, fmt_name, trans_b, true);
    CheckGroups(gs, s.e);
    TORCH_CHECK(s.n % 2 == 0 && (ofmt != CCH_FMT_E2M1 || s.n % 4 == 0), "n must be even (a multiple of 4 for FP4 output)");
    const int64_t h = s.n / 2;
    at::Tensor payload = Bytes(a, {s.t, ofmt == CCH_FMT_E2M1 ? h / 2 : h}), scales = Bytes(a, {s.t, ScaleCols(h)});
    Check(cch_mx_gmm_swiglu_mx(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), gs.data_ptr<int32_t>(), payload.data_ptr(), scales.data_ptr(), s.e,
                               s.t, s.n, s.k, s.fmt, (int)trans_b, ofmt, StreamOf(a)),
          "mx_grouped_matmul_swiglu_mx");
    return {payload, scales};
}

// The MXFP8 MoE FFN of one rank that holds every expert, routing to combine (the reference's
// Ascend950DispatchFFNCombine, examples/ascend950_dispatch_ffn_combine/ascend950_dispatch_ffn_combine_device.h:124-176):
// routing sort -> MXFP8 quantise-and-scatter -> GMM1 + SwiGLU + MXFP8 quantise -> GMM2 -> weighted un-permute.
at::Tensor MoeFfnMxfp8(const at::Tensor &x_in, const at::Tensor &expert_idx_in, const at::Tensor &probs_in, const at::Tensor &w1_in, const at::Tensor &sw1_in,
                       const at::Tensor &w2_in, const at::Tensor &sw2_in, int64_t trans_b)
{
    NeedInit();
    TORCH_CHECK(x_in.dim() == 2 && x_in.scalar_type() == at::kBFloat16, "x must be a 2-D bfloat16 tensor");
    TORCH_CHECK(expert_idx_in.dim() == 2 && expert_idx_in.size(0) == x_in.size(0) && expert_idx_in.scalar_type() == at::kInt,
                "expert_idx must be an int32 [m, top_k] tensor");
    TORCH_CHECK(probs_in.sizes() == expert_idx_in.sizes() && probs_in.scalar_type() == at::kFloat, "probs must be a float32 [m, top_k] tensor");
    TORCH_CHECK(w1_in.dim() == 3 && w2_in.dim() == 3 && w1_in.size(0) == w2_in.size(0), "w1 and w2 must hold one matrix per expert");
    SameDevice("moe_ffn_mxfp8", {{"x", x_in}, {"expert_idx", expert_idx_in}, {"probs", probs_in}, {"w1", w1_in}, {"sw1", sw1_in}, {"w2", w2_in}, {"sw2", sw2_in}});
    c10::DeviceGuard guard(x_in.device());
    const at::Tensor x = x_in.contiguous(), idx = expert_idx_in.contiguous(), probs = probs_in.contiguous();
    const at::Tensor w1 = w1_in.contiguous(), sw1 = sw1_in.contiguous(), w2 = w2_in.contiguous(), sw2 = sw2_in.contiguous();
    const int64_t m = x.size(0), k = x.size(1), top_k = idx.size(1), rows = m * top_k, e = w1.size(0);
    const int64_t n = trans_b ? w1.size(1) : w1.size(2), h = n / 2;
    TORCH_CHECK((trans_b ? w1.size(2) : w1.size(1)) == k && n % 2 == 0, "w1 must be [E, k, n] (trans_b: [E, n, k]) with n even");
    TORCH_CHECK((trans_b ? w2.size(2) : w2.size(1)) == h && (trans_b ? w2.size(1) : w2.size(2)) == k, "w2 must be [E, n/2, k] (trans_b: [E, k, n/2])");
    TORCH_CHECK(sw1.numel() == e * ScaleCols(k) * n && sw2.numel() == e * ScaleCols(h) * k, "scale tensors do not match the weights");
    void *stream = StreamOf(x);
    const auto i32 = x.options().dtype(at::kInt);
    at::Tensor d2s = at::empty({rows}, i32), s2d = at::empty({rows}, i32), cnt = at::empty({e}, i32);
    const int64_t ws_bytes = std::max<int64_t>(cch_moe_init_routing_workspace_bytes(rows, (int)e), 4);
    at::Tensor ws = Bytes(x, {ws_bytes});
    Check(cch_moe_init_routing(idx.data_ptr<int32_t>(), rows, (int)e, d2s.data_ptr<int32_t>(), s2d.data_ptr<int32_t>(), cnt.data_ptr<int32_t>(), 0,
                               ws.data_ptr(), ws_bytes, stream),
          "moe_ffn_mxfp8 (routing)");
    at::Tensor packed = Bytes(x, {rows, k + ScaleCols(k)});
    Check(cch_mx_quant_scatter_packed_rows(x.data_ptr(), s2d.data_ptr<int32_t>(), packed.data_ptr(), rows, m, k, (int)top_k, CCH_FMT_E4M3, CCH_ROUND_RNE, stream),
          "moe_ffn_mxfp8 (dispatch)");
    at::Tensor act = Bytes(x, {rows, h}), act_scales = Bytes(x, {rows, ScaleCols(h)});
    Check(cch_mx_gmm_swiglu_mx_packed(packed.data_ptr(), w1.data_ptr(), sw1.data_ptr(), cnt.data_ptr<int32_t>(), act.data_ptr(), act_scales.data_ptr(), e, rows,
                                      n, k, CCH_FMT_E4M3, (int)trans_b, CCH_FMT_E4M3, stream),
          "moe_ffn_mxfp8 (up projection)");
    at::Tensor y = at::empty({rows, k}, x.options());
    Check(cch_mx_gmm(act.data_ptr(), act_scales.data_ptr(), w2.data_ptr(), sw2.data_ptr(), cnt.data_ptr<int32_t>(), y.data_ptr(), e, rows, k, h, CCH_FMT_E4M3,
                     (int)trans_b, stream),
          "moe_ffn_mxfp8 (down projection)");
    at::Tensor out = at::empty({m, k}, x.options());
    Check(cch_moe_token_unpermute(y.data_ptr(), s2d.data_ptr<int32_t>(), probs.data_ptr<float>(), out.data_ptr(), rows, m, k, (int)top_k, stream),
          "moe_ffn_mxfp8 (combine)");
    return out;
}

// ---------------------------------------------------------------------------------------------
// Meta kernels: output shapes only (reference torch_bindings_meta.cpp:18-30 returns at::empty_symint of the result shape)

c10::SymInt SymScaleCols(const c10::SymInt &k) { return ((k + 63) / 64) * 2; }

at::Tensor MetaEmpty(const at::Tensor &like, c10::SymIntArrayRef shape, at::ScalarType dtype)
{
    return at::empty_symint(shape, like.options().dtype(dtype));
}

std::tuple<at::Tensor, at::Tensor> MxQuantMeta(const at::Tensor &x, std::string fmt_name, int64_t)
{
    const int fmt = FormatCode(fmt_name);
    const c10::SymInt m = x.sym_size(0), k = x.sym_size(1);
    return {MetaEmpty(x, {m, IsFp4(fmt) ? (k + 1) / 2 : k}, at::kByte), MetaEmpty(x, {m, SymScaleCols(k)}, at::kByte)};
}

c10::SymInt MxN(const at::Tensor &b, int first, int fmt, int64_t trans_b)
{
    return trans_b ? b.sym_size(first) : b.sym_size(first + 1) * (IsFp4(fmt) ? 2 : 1);
}

at::Tensor W8A8Meta(const at::Tensor &a, const at::Tensor &b, const at::Tensor &, const at::Tensor &, int64_t trans_b)
{
    return MetaEmpty(a, {a.sym_size(0), trans_b ? b.sym_size(0) : b.sym_size(1)}, at::kBFloat16);
}

at::Tensor MxMatmulMeta(const at::Tensor &a, const at::Tensor &, const at::Tensor &b, const at::Tensor &, std::string fmt_name, int64_t trans_b)
{
    return MetaEmpty(a, {a.sym_size(0), MxN(b, 0, FormatCode(fmt_name), trans_b)}, at::kBFloat16);
}

at::Tensor GmmSwigluMeta(const at::Tensor &x, const at::Tensor &w, const at::Tensor &, const at::Tensor &, const at::Tensor &, int64_t trans_b)
{
    return MetaEmpty(x, {x.sym_size(0), (trans_b ? w.sym_size(1) : w.sym_size(2)) / 2}, at::kBFloat16);
}

std::tuple<at::Tensor, at::Tensor> GmmSwigluMxMeta(const at::Tensor &x, const at::Tensor &w, const at::Tensor &, const at::Tensor &, const at::Tensor &,
                                                   int64_t trans_b, std::string fmt_name)
{
    const c10::SymInt h = (trans_b ? w.sym_size(1) : w.sym_size(2)) / 2;
    return {MetaEmpty(x, {x.sym_size(0), IsFp4(FormatCode(fmt_name)) ? h / 2 : h}, at::kByte), MetaEmpty(x, {x.sym_size(0), SymScaleCols(h)}, at::kByte)};
}

at::Tensor MxGmmMeta(const at::Tensor &a, const at::Tensor &, const at::Tensor &b, const at::Tensor &, const at::Tensor &, std::string fmt_name, int64_t trans_b)
{
    return MetaEmpty(a, {a.sym_size(0), MxN(b, 1, FormatCode(fmt_name), trans_b)}, at::kBFloat16);
}

std::tuple<at::Tensor, at::Tensor> MxGmmSwigluMxMeta(const at::Tensor &a, const at::Tensor &, const at::Tensor &b, const at::Tensor &, const at::Tensor &,
                                                     std::string fmt_name, int64_t trans_b, std::string out_fmt_name)
{
    const c10::SymInt h = MxN(b, 1, FormatCode(fmt_name), trans_b) / 2;
    return {MetaEmpty(a, {a.sym_size(0), IsFp4(FormatCode(out_fmt_name)) ? h / 2 : h}, at::kByte), MetaEmpty(a, {a.sym_size(0), SymScaleCols(h)}, at::kByte)};
}

at::Tensor MoeFfnMeta(const at::Tensor &x, const at::Tensor &, const at::Tensor &, const at::Tensor &, const at::Tensor &, const at::Tensor &,
                      const at::Tensor &, int64_t)
{
    return MetaEmpty(x, x.sym_sizes(), x.scalar_type());
}

}  // namespace

TORCH_LIBRARY(catccos, m)
{
    m.def("init(int rank_id, int rank_size, int local_mem_size, str ip_port) -> int");
    m.def("finalize() -> int");
    m.def("mx_quant(Tensor x, str fmt, int rounding) -> (Tensor, Tensor)");
    m.def("w8a8_matmul_dequant(Tensor a, Tensor b, Tensor per_tok, Tensor per_ch, int trans_b) -> Tensor");
    m.def("mx_matmul(Tensor a, Tensor sa, Tensor b, Tensor sb, str fmt, int trans_b) -> Tensor");
    m.def("gmm_dequant_swiglu(Tensor x, Tensor w, Tensor group_sizes, Tensor per_tok, Tensor per_ch, int trans_b) -> Tensor");
    m.def("mx_grouped_matmul(Tensor a, Tensor sa, Tensor b, Tensor sb, Tensor group_sizes, str fmt, int trans_b) -> Tensor");
    m.def("mx_grouped_matmul_swiglu_mx(Tensor a, Tensor sa, Tensor b, Tensor sb, Tensor group_sizes, str fmt, int trans_b, str out_fmt) -> (Tensor, Tensor)");
    m.def("gmm_dequant_swiglu_mx(Tensor x, Tensor w, Tensor group_sizes, Tensor per_tok, Tensor per_ch, int trans_b, str fmt) -> (Tensor, Tensor)");
    m.def("moe_ffn_mxfp8(Tensor x, Tensor expert_idx, Tensor probs, Tensor w1, Tensor sw1, Tensor w2, Tensor sw2, int trans_b) -> Tensor");
}

// init / finalize take no tensors: one kernel for every backend, as in the reference (torch_bindings.cpp:233-238)
TORCH_LIBRARY_IMPL(catccos, CompositeExplicitAutograd, m)
{
    m.impl("init", &Init);
    m.impl("finalize", &Finalize);
}

// the GPU key (HIP devices answer to it in a ROCm build of PyTorch); CPU tensors find no kernel
TORCH_LIBRARY_IMPL(catccos, CUDA, m)
{
    m.impl("mx_quant", &MxQuant);
    m.impl("w8a8_matmul_dequant", &W8A8MatmulDequant);
    m.impl("mx_matmul", &MxMatmul);
    m.impl("gmm_dequant_swiglu", &GmmDequantSwiglu);
    m.impl("mx_grouped_matmul", &MxGroupedMatmul);
    m.impl("mx_grouped_matmul_swiglu_mx", &MxGroupedMatmulSwigluMx);
    m.impl("gmm_dequant_swiglu_mx", &GmmDequantSwigluMx);
    m.impl("moe_ffn_mxfp8", &MoeFfnMxfp8);
}

TORCH_LIBRARY_IMPL(catccos, Meta, m)
{
    m.impl("mx_quant", &MxQuantMeta);
    m.impl("w8a8_matmul_dequant", &W8A8Meta);
    m.impl("mx_matmul", &MxMatmulMeta);
    m.impl("gmm_dequant_swiglu", &GmmSwigluMeta);
    m.impl("mx_grouped_matmul", &MxGmmMeta);
    m.impl("mx_grouped_matmul_swiglu_mx", &MxGmmSwigluMxMeta);
    m.impl("gmm_dequant_swiglu_mx", &GmmSwigluMxMeta);
    m.impl("moe_ffn_mxfp8", &MoeFfnMeta);
}
