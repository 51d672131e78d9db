// PyTorch extension over the C ABI of libsbvr_hip.so: the operators that the
// reference binds in sbvr/kernels/sbvr_ops.cpp:152-172 (`_sbvr_mm_T`,
// `_sbvr_row_deq_mm_T`, `_sbvr_cuda_init`), with the same argument lists and the
// same shape inference from tensor sizes (:44-51, :90-96), plus the fp16
// activation linear over the default layout and its two one-row variants.
// This file holds no device code; it is the only C++ here that sees at::Tensor.
// Unlike the reference's wrappers it checks device, dtype and contiguity, guards
// the device and launches on torch's current HIP stream.  sbvr/hip.py offers the
// same operators through ctypes; both call the same entry points.
#include <torch/extension.h>

// (PyTorch on ROCm labels HIP devices "cuda"; these are the guard and stream types that accept that label)
#include <ATen/hip/HIPContext.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <map>
#include <mutex>
#include <tuple>
#include <vector>

#include "../../include/sbvr_hip.h"

namespace {

using DeviceGuard = c10::hip::HIPGuardMasqueradingAsCUDA;

hipStream_t current_stream()
{
    return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream();
}

void want(const torch::Tensor &t, const char *name, c10::ScalarType dtype, int64_t dim, const torch::Tensor *like)
{
    TORCH_CHECK(t.is_cuda(), name, " must be on a GPU (got ", t.device(), "); there is no CPU path");
    TORCH_CHECK(t.scalar_type() == dtype, name, " must have dtype ", dtype, ", got ", t.scalar_type());
    TORCH_CHECK(t.dim() == dim, name, " must have ", dim, " dimensions, got ", t.dim());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    if (like)
        TORCH_CHECK(t.device() == like->device(), name, " is on ", t.device(), ", expected ", like->device());
}

// uint8 indices for up to 256 lines, uint16 beyond (sbvr_kernel.cu:931-932)
int idx_bytes(const torch::Tensor &idx, int64_t lines, const char *name, const torch::Tensor &like)
{
    const auto expect = lines <= 256 ? torch::kUInt8 : torch::kUInt16;
    want(idx, name, expect, 2, &like);
    return lines <= 256 ? 1 : 2;
}

// the bias is used only when its length is N (sbvr_ops.cpp:56-58)
// (None is accepted beside the reference's 0-length tensor for "no bias")
using Bias = c10::optional<torch::Tensor>;

const void *bias_ptr(const Bias &bias, int64_t n, const torch::Tensor &like)
{
    if (!bias.has_value() || !bias->defined() || bias->numel() == 0 || bias->size(0) != n)
        return nullptr;
    want(*bias, "bias", torch::kFloat16, 1, &like);
    return bias->data_ptr();
}

void check(int rc)
{
    TORCH_CHECK(rc == SBVR_HIP_OK, "libsbvr_hip: error ", rc, ": ", sbvr_hip_last_error());
}

// Zero-initialised split-K accumulators per (device, stream), grown on demand; the kernels
// leave the part that must be zero zeroed.  A buffer that is outgrown is kept until the process
// ends: a HIP graph captured earlier on that stream still holds its address.
torch::Tensor workspace(size_t nbytes, const torch::Tensor &like, hipStream_t stream)
{
    static std::mutex mu;
    static std::map<std::tuple<int, hipStream_t>, torch::Tensor> held;
    static std::vector<torch::Tensor> outgrown;
    std::lock_guard<std::mutex> lock(mu);
    auto key = std::make_tuple(static_cast<int>(like.get_device()), stream);
    auto it = held.find(key);
    if (it == held.end() || static_cast<size_t>(it->second.numel()) < nbytes) {
        if (it != held.end())
            outgrown.push_back(it->second);
        const int64_t size = static_cast<int64_t>(nbytes > (1u << 20) ? nbytes : (1u << 20));
        held[key] = torch::zeros({size}, torch::dtype(torch::kUInt8).device(like.device()));
        it = held.find(key);
    }
    return it->second;
}

struct LinearShape {
    int64_t M, N, K, S, G, L;
    int ib;
};

LinearShape linear_shape(int64_t M, int64_t K, const torch::Tensor &bvr, const torch::Tensor &coeff_idx,
                         const torch::Tensor &coeff_cache, int64_t bvr_len, const torch::Tensor &like)
{
    want(bvr, "bvr", torch::kUInt32, 3, &like);
    want(coeff_cache, "coeff_cache", torch::kFloat16, 2, &like);
    LinearShape s{};
    s.M = M;
    s.K = K;
    s.N = bvr.size(1);
    s.S = bvr.size(2);
    s.L = coeff_cache.size(0);
    s.ib = idx_bytes(coeff_idx, s.L, "coeff_idx", like);
    TORCH_CHECK(bvr.size(0) * 32 == K, "x has K=", K, " but bvr holds ", bvr.size(0) * 32, " columns");
    TORCH_CHECK(coeff_idx.size(1) == s.N && coeff_cache.size(1) == s.S, "coeff_idx / coeff_cache shapes do not match bvr");
    s.G = bvr_len > 0 ? bvr_len : K / coeff_idx.size(0);
    TORCH_CHECK(s.G * coeff_idx.size(0) == K, "coeff_idx has ", coeff_idx.size(0), " groups, K=", K, ", bvr_len=", s.G);
    return s;
}

}  // namespace

// Counterpart of sbvr_cuda_init (sbvr_ops.cpp:122-150): checks that the current device is a gfx950 part.
void sbvr_hip_init_current()
{
    check(sbvr_hip_init(static_cast<int>(at::hip::current_device())));
}

// y = x @ decode(W)^T (+ bias): x (M, K) fp16; W in the default layout, bvr (K/32, N, S) uint32,
// coeff_idx (K/G, N), coeff_cache (L, S) fp16.  bvr_len <= 0: the group length follows from coeff_idx.
// out: an (M, N) fp16 tensor to write into (a caller that records a HIP graph brings its own), or None.
torch::Tensor sbvr_linear_f16(torch::Tensor x, torch::Tensor bvr, torch::Tensor coeff_idx, torch::Tensor coeff_cache,
                              Bias bias, int64_t bvr_len, int64_t flags, c10::optional<torch::Tensor> out_opt)
{
    want(x, "x", torch::kFloat16, 2, nullptr);
    const LinearShape s = linear_shape(x.size(0), x.size(1), bvr, coeff_idx, coeff_cache, bvr_len, x);
    const DeviceGuard guard(x.device());
    hipStream_t stream = current_stream();
    torch::Tensor out;
    if (out_opt.has_value() && out_opt->defined()) {
        out = *out_opt;
        want(out, "out", torch::kFloat16, 2, &x);
        TORCH_CHECK(out.size(0) == s.M && out.size(1) == s.N, "out has the wrong shape");
    } else {
        out = torch::empty({s.M, s.N}, torch::dtype(torch::kFloat16).device(x.device()));
    }
    const size_t need = sbvr_hip_linear_f16_workspace(s.M, s.N, s.K, s.S, s.G);
    torch::Tensor ws = need ? workspace(need, x, stream) : torch::Tensor();
    check(sbvr_hip_linear_f16(x.data_ptr(), static_cast<const uint32_t *>(bvr.data_ptr()), coeff_idx.data_ptr(), s.ib,
                              coeff_cache.data_ptr(), bias_ptr(bias, s.N, x), out.data_ptr(), s.M, s.N, s.K, s.S, s.G,
                              s.L, need ? ws.data_ptr() : nullptr, need ? ws.numel() : 0, static_cast<int>(flags), stream));
    return out;
}

// The linear of fp16(fp16(silu(gate)) * up) for gate_up (1, 2K) = gate | up.
torch::Tensor sbvr_linear_f16_swiglu(torch::Tensor gate_up, torch::Tensor bvr, torch::Tensor coeff_idx,
                                     torch::Tensor coeff_cache, Bias bias, int64_t bvr_len)
{
    want(gate_up, "gate_up", torch::kFloat16, 2, nullptr);
    TORCH_CHECK(gate_up.size(1) % 2 == 0, "gate_up must have an even number of columns");
    const LinearShape s = linear_shape(gate_up.size(0), gate_up.size(1) / 2, bvr, coeff_idx, coeff_cache, bvr_len, gate_up);
    const DeviceGuard guard(gate_up.device());
    hipStream_t stream = current_stream();
    auto out = torch::empty({s.M, s.N}, torch::dtype(torch::kFloat16).device(gate_up.device()));
    const size_t need = sbvr_hip_linear_f16_workspace(s.M, s.N, s.K, s.S, s.G);
    torch::Tensor ws = need ? workspace(need, gate_up, stream) : torch::Tensor();
    check(sbvr_hip_linear_f16_swiglu(gate_up.data_ptr(), static_cast<const uint32_t *>(bvr.data_ptr()), coeff_idx.data_ptr(),
                                     s.ib, coeff_cache.data_ptr(), bias_ptr(bias, s.N, gate_up), out.data_ptr(), s.M, s.N,
                                     s.K, s.S, s.G, s.L, need ? ws.data_ptr() : nullptr, need ? ws.numel() : 0, stream));
    return out;
}

// x_out <- r = fp16(x + delta); returns the linear of norm_weight * fp16(r * rsqrt(mean(r^2) + eps)).
torch::Tensor sbvr_linear_f16_add_rmsnorm(torch::Tensor x, torch::Tensor delta, torch::Tensor norm_weight, double eps,
                                          torch::Tensor x_out, torch::Tensor bvr, torch::Tensor coeff_idx,
                                          torch::Tensor coeff_cache, Bias bias, int64_t bvr_len)
{
    want(x, "x", torch::kFloat16, 2, nullptr);
    want(delta, "delta", torch::kFloat16, 2, &x);
    want(x_out, "x_out", torch::kFloat16, 2, &x);
    want(norm_weight, "norm_weight", torch::kFloat16, 1, &x);
    TORCH_CHECK(x.size(0) == 1 && delta.sizes() == x.sizes() && x_out.sizes() == x.sizes() &&
                    norm_weight.size(0) == x.size(1),
                "x, delta and x_out must be (1, K) and norm_weight (K)");
    const LinearShape s = linear_shape(1, x.size(1), bvr, coeff_idx, coeff_cache, bvr_len, x);
    const DeviceGuard guard(x.device());
    hipStream_t stream = current_stream();
    auto out = torch::empty({1, s.N}, torch::dtype(torch::kFloat16).device(x.device()));
    const size_t need = sbvr_hip_linear_f16_workspace(1, s.N, s.K, s.S, s.G);
    torch::Tensor ws = need ? workspace(need, x, stream) : torch::Tensor();
    check(sbvr_hip_linear_f16_add_rmsnorm(x.data_ptr(), delta.data_ptr(), norm_weight.data_ptr(), static_cast<float>(eps),
                                          x_out.data_ptr(), static_cast<const uint32_t *>(bvr.data_ptr()),
                                          coeff_idx.data_ptr(), s.ib, coeff_cache.data_ptr(), bias_ptr(bias, s.N, x),
                                          out.data_ptr(), s.N, s.K, s.S, s.G, s.L, need ? ws.data_ptr() : nullptr,
                                          need ? ws.numel() : 0, stream));
    return out;
}

// Both operands encoded, default layout: l_bvr (K/32, M, Sl), r_bvr (K/32, N, Sr) (sbvr_ops.cpp:35-76).
torch::Tensor sbvr_mm_T(torch::Tensor l_bvr, torch::Tensor l_coeff_idx, torch::Tensor l_coeff_cache, torch::Tensor r_bvr,
                        torch::Tensor r_coeff_idx, torch::Tensor r_coeff_cache, Bias bias)
{
    want(l_bvr, "l_bvr", torch::kUInt32, 3, nullptr);
    want(r_bvr, "r_bvr", torch::kUInt32, 3, &l_bvr);
    want(l_coeff_cache, "l_coeff_cache", torch::kFloat16, 2, &l_bvr);
    want(r_coeff_cache, "r_coeff_cache", torch::kFloat16, 2, &l_bvr);
    const int64_t M = l_bvr.size(1), N = r_bvr.size(1), K = l_bvr.size(0) * 32;
    const int64_t Sl = l_bvr.size(2), Sr = r_bvr.size(2), Ll = l_coeff_cache.size(0), Lr = r_coeff_cache.size(0);
    TORCH_CHECK(l_bvr.size(0) == r_bvr.size(0), "operands disagree on K: ", K, " vs ", r_bvr.size(0) * 32);
    const int lib = idx_bytes(l_coeff_idx, Ll, "l_coeff_idx", l_bvr), rib = idx_bytes(r_coeff_idx, Lr, "r_coeff_idx", l_bvr);
    TORCH_CHECK(l_coeff_idx.size(1) == M && r_coeff_idx.size(1) == N && l_coeff_idx.size(0) == r_coeff_idx.size(0) &&
                    l_coeff_cache.size(1) == Sl && r_coeff_cache.size(1) == Sr,
                "index / table shapes do not match the bit planes");
    const int64_t G = K / l_coeff_idx.size(0);
    TORCH_CHECK(G * l_coeff_idx.size(0) == K, "coeff_idx has ", l_coeff_idx.size(0), " groups, K=", K);
    const DeviceGuard guard(l_bvr.device());
    auto out = torch::empty({M, N}, torch::dtype(torch::kFloat16).device(l_bvr.device()));
    hipStream_t stream = current_stream();
    const size_t need = sbvr_hip_mm_T_workspace(static_cast<int>(M), static_cast<int>(N));
    torch::Tensor ws;                    // (no split of K for this call: no workspace, nothing allocated)
    if (need)
        ws = workspace(need, l_bvr, stream);
    check(sbvr_hip_mm_T_ws(static_cast<const uint32_t *>(l_bvr.data_ptr()), l_coeff_idx.data_ptr(), lib,
                           l_coeff_cache.data_ptr(), static_cast<const uint32_t *>(r_bvr.data_ptr()), r_coeff_idx.data_ptr(),
                           rib, r_coeff_cache.data_ptr(), bias_ptr(bias, N, l_bvr), out.data_ptr(), M, N, K, Sl, Sr, G, Ll,
                           Lr, need ? ws.data_ptr() : nullptr, need, stream));
    return out;
}

// fp16 l_w (M, K) against a trans=True weight: r_bvr (N/32, K, S), r_coeff_idx (N/G, K) (sbvr_ops.cpp:79-120).
// use_shfl chose between equivalent CUDA kernels in the reference and is ignored.
torch::Tensor sbvr_row_deq_mm_T(torch::Tensor l_w, torch::Tensor r_bvr, torch::Tensor r_coeff_idx,
                                torch::Tensor r_coeff_cache, Bias bias, int64_t use_shfl)
{
    (void)use_shfl;
    want(l_w, "l_w", torch::kFloat16, 2, nullptr);
    want(r_bvr, "r_bvr", torch::kUInt32, 3, &l_w);
    want(r_coeff_cache, "r_coeff_cache", torch::kFloat16, 2, &l_w);
    const int64_t M = l_w.size(0), K = l_w.size(1), N = r_bvr.size(0) * 32, S = r_bvr.size(2), L = r_coeff_cache.size(0);
    const int ib = idx_bytes(r_coeff_idx, L, "r_coeff_idx", l_w);
    TORCH_CHECK(r_bvr.size(1) == K && r_coeff_idx.size(1) == K && r_coeff_cache.size(1) == S, "operand shapes do not match");
    const int64_t G = N / r_coeff_idx.size(0);
    TORCH_CHECK(G * r_coeff_idx.size(0) == N, "r_coeff_idx has ", r_coeff_idx.size(0), " groups, N=", N);
    const DeviceGuard guard(l_w.device());
    auto out = torch::empty({M, N}, torch::dtype(torch::kFloat16).device(l_w.device()));
    hipStream_t stream = current_stream();
    const size_t need = sbvr_hip_row_deq_mm_T_workspace(static_cast<int>(M), static_cast<int>(N));
    torch::Tensor ws;                    // (no split of K for this call: no workspace, nothing allocated)
    if (need)
        ws = workspace(need, l_w, stream);
    check(sbvr_hip_row_deq_mm_T_ws(l_w.data_ptr(), static_cast<const uint32_t *>(r_bvr.data_ptr()), r_coeff_idx.data_ptr(), ib,
                                   r_coeff_cache.data_ptr(), bias_ptr(bias, N, l_w), out.data_ptr(), M, N, K, S, G, L,
                                   need ? ws.data_ptr() : nullptr, need, stream));
    return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    namespace py = pybind11;
    m.def("_sbvr_hip_init", &sbvr_hip_init_current, "Checks that the current device is a gfx950 part");
    m.def("_sbvr_cuda_init", &sbvr_hip_init_current, "Alias of _sbvr_hip_init under the reference's name");
    m.def("_sbvr_mm_T", &sbvr_mm_T, "SBVR x SBVR^T, both operands encoded", py::arg("l_bvr"), py::arg("l_coeff_idx"),
          py::arg("l_coeff_cache"), py::arg("r_bvr"), py::arg("r_coeff_idx"), py::arg("r_coeff_cache"), py::arg("bias"));
    m.def("_sbvr_row_deq_mm_T", &sbvr_row_deq_mm_T, "fp16 x SBVR^T over the trans=True layout", py::arg("l_w"),
          py::arg("r_bvr"), py::arg("r_coeff_idx"), py::arg("r_coeff_cache"), py::arg("bias"), py::arg("use_shfl") = 0);
    m.def("_sbvr_linear_f16", &sbvr_linear_f16, "fp16 x SBVR^T over the default layout", py::arg("x"), py::arg("bvr"),
          py::arg("coeff_idx"), py::arg("coeff_cache"), py::arg("bias") = py::none(), py::arg("bvr_len") = 0,
          py::arg("flags") = 0, py::arg("out") = py::none());
    m.def("last_kernel", &sbvr_hip_last_kernel, "which kernel the last linear call of this thread launched");
    m.def("_sbvr_linear_f16_swiglu", &sbvr_linear_f16_swiglu, "the linear of silu(gate) * up, one row", py::arg("gate_up"),
          py::arg("bvr"), py::arg("coeff_idx"), py::arg("coeff_cache"), py::arg("bias") = py::none(),
          py::arg("bvr_len") = 0);
    m.def("_sbvr_linear_f16_add_rmsnorm", &sbvr_linear_f16_add_rmsnorm, "x_out <- x + delta, the linear of its RMSNorm",
          py::arg("x"), py::arg("delta"), py::arg("norm_weight"), py::arg("eps"), py::arg("x_out"), py::arg("bvr"),
          py::arg("coeff_idx"), py::arg("coeff_cache"), py::arg("bias") = py::none(), py::arg("bvr_len") = 0);
    m.def("version", &sbvr_hip_version, "ABI version of the library underneath");
}
