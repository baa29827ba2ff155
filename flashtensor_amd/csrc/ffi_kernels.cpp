// pybind11 module `ft_ffi` over the C ABI of include/ft_abi.h, in the idiom of the reference's ffi/ layer:
// one extension module whose sub-modules are filled by init_ffi_* functions (ffi/ffi.cpp:3-7, ffi/ffi.h:12-14),
// C++ exceptions for errors (std::runtime_error as in ffi/passes.cpp:81-83, std::invalid_argument for bad
// arguments), device pointers crossing as integers (tensor.data_ptr(), the way the reference's TensorRT closure
// hands them to set_tensor_address, python/asuka/backend/tensorrt/builder.py:112-119).  To graft it onto the
// reference itself: add `void init_ffi_kernels(py::module_ &&m);` to ffi/ffi.h and
// `init_ffi_kernels(m.def_submodule("kernels"));` to ffi/ffi.cpp, and link libflashtensor_hip.so.
//
// Unlike the reference's bindings (which hold the GIL throughout), every launch releases the GIL: the calls only
// queue kernels and touch no Python object.  No torch headers are needed.
#include <pybind11/pybind11.h>

#include <cstdint>
#include <stdexcept>
#include <string>

#include "../../include/ft_abi.h"

namespace py = pybind11;

namespace {

// ft_last_error() is thread-local: read it on the calling thread, before the GIL is taken back.
void check(int rc) {
  if (rc == FT_OK) return;
  const std::string msg = std::string("libflashtensor_hip: ") + ft_last_error() + " (status " + std::to_string(rc) + ")";
  if (rc == FT_EINVAL) throw std::invalid_argument(msg);
  throw std::runtime_error(msg);
}

template <typename T>
T* ptr(uintptr_t p) {
  return reinterpret_cast<T*>(p);
}

FtStrides strides(const py::tuple& t) {
  if (t.size() != 3) throw std::invalid_argument("strides need 3 entries (batch, sequence, head)");
  return FtStrides{t[0].cast<int64_t>(), t[1].cast<int64_t>(), t[2].cast<int64_t>()};
}

}  // namespace

void init_ffi_kernels(py::module_&& m) {
  m.doc() = "fused attention-variant kernels for MI355X (C ABI of include/ft_abi.h)";
  m.attr("ABI_VERSION") = FT_ABI_VERSION;
  m.attr("OK") = (int)FT_OK;
  m.attr("EINVAL") = (int)FT_EINVAL;
  m.attr("EUNSUPPORTED") = (int)FT_EUNSUPPORTED;
  m.attr("ELAUNCH") = (int)FT_ELAUNCH;
  m.attr("EWORKSPACE") = (int)FT_EWORKSPACE;
  m.attr("F16") = (int)FT_F16;
  m.attr("BF16") = (int)FT_BF16;
  m.attr("F32") = (int)FT_F32;
  m.attr("CAUSAL") = (unsigned)FT_CAUSAL;
  m.attr("FAST_LOGITS") = (unsigned)FT_FAST_LOGITS;
  m.attr("OP_ATTN") = (int)FT_OP_ATTN;
  m.attr("OP_COLSTATS") = (int)FT_OP_COLSTATS;
  m.attr("OP_KEYFORMER") = (int)FT_OP_KEYFORMER;
  m.attr("OP_EA") = (int)FT_OP_EA;
  m.attr("OP_SIMA") = (int)FT_OP_SIMA;
  m.attr("OP_CORM") = (int)FT_OP_CORM;
  m.attr("STATIC_SCRATCH_BYTES") = (size_t)FT_STATIC_SCRATCH_BYTES;

  py::class_<FtAttnArgs>(m, "AttnArgs", py::module_local())
      .def(py::init([](uintptr_t q, uintptr_t k, uintptr_t v, uintptr_t o, py::tuple sq, py::tuple sk, py::tuple sv, py::tuple so,
                       int B, int H, int Sq, int Skv, int D, int dtype, unsigned flags, int Hkv) {
             return FtAttnArgs{ptr<const void>(q), ptr<const void>(k), ptr<const void>(v), ptr<void>(o), strides(sq), strides(sk),
                               strides(sv), strides(so), B, H, Sq, Skv, D, dtype, flags, Hkv};
           }),
           py::arg("q"), py::arg("k"), py::arg("v"), py::arg("o"), py::arg("sq"), py::arg("sk"), py::arg("sv"), py::arg("so"),
           py::arg("B"), py::arg("H"), py::arg("Sq"), py::arg("Skv"), py::arg("D"), py::arg("dtype"), py::arg("flags") = 0u,
           py::arg("Hkv") = 0)
      .def_readwrite("B", &FtAttnArgs::B)
      .def_readwrite("H", &FtAttnArgs::H)
      .def_readwrite("Sq", &FtAttnArgs::Sq)
      .def_readwrite("Skv", &FtAttnArgs::Skv)
      .def_readwrite("D", &FtAttnArgs::D)
      .def_readwrite("dtype", &FtAttnArgs::dtype)
      .def_readwrite("flags", &FtAttnArgs::flags)
      .def_readwrite("Hkv", &FtAttnArgs::Hkv);

  py::class_<FtNoise>(m, "Noise", py::module_local())
      .def(py::init([](uintptr_t exp_rand, int64_t stride_b, int64_t stride_h, int64_t stride_row, uint64_t seed) {
             return FtNoise{ptr<const float>(exp_rand), stride_b, stride_h, stride_row, seed};
           }),
           py::arg("exp_rand") = 0, py::arg("stride_b") = 0, py::arg("stride_h") = 0, py::arg("stride_row") = 0, py::arg("seed") = 0);

  py::class_<FtLinBlockArgs>(m, "LinBlockArgs", py::module_local())
      .def(py::init([](uintptr_t x, uintptr_t w_qkv, uintptr_t b_qkv, uintptr_t w_out, uintptr_t b_out, uintptr_t y, int B, int S, int H,
                       int D, int dtype) {
             return FtLinBlockArgs{ptr<const void>(x), ptr<const void>(w_qkv), ptr<const void>(b_qkv), ptr<const void>(w_out),
                                   ptr<const void>(b_out), ptr<void>(y), B, S, H, D, dtype};
           }),
           py::arg("x"), py::arg("w_qkv"), py::arg("b_qkv"), py::arg("w_out"), py::arg("b_out"), py::arg("y"), py::arg("B"),
           py::arg("S"), py::arg("H"), py::arg("D"), py::arg("dtype"));

  m.def("abi_version", [] { return ft_abi_version(); });
  m.def("last_error", [] { return std::string(ft_last_error()); });
  m.def("workspace_bytes", [](int op, const FtAttnArgs& a) { return ft_workspace_bytes(op, &a); });

  m.def("attn_fwd", [](const FtAttnArgs& a, uintptr_t lse, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_attn_fwd(&a, ptr<float>(lse), ptr<void>(stream)));
  }, py::arg("args"), py::arg("lse") = 0, py::arg("stream") = 0);

  m.def("attn_colstats_fwd", [](const FtAttnArgs& a, uintptr_t colsum, uintptr_t colsumsq, uintptr_t ws, size_t ws_bytes, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_attn_colstats_fwd(&a, ptr<float>(colsum), ptr<float>(colsumsq), ptr<void>(ws), ws_bytes, ptr<void>(stream)));
  }, py::arg("args"), py::arg("colsum"), py::arg("colsumsq"), py::arg("workspace"), py::arg("workspace_bytes"), py::arg("stream") = 0);

  m.def("attn_colstats_fwd_static", [](const FtAttnArgs& a, uintptr_t colsum, uintptr_t colsumsq, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_attn_colstats_fwd_static(&a, ptr<float>(colsum), ptr<float>(colsumsq), ptr<void>(stream)));
  }, py::arg("args"), py::arg("colsum"), py::arg("colsumsq") = 0, py::arg("stream") = 0);

  m.def("keyformer_fwd", [](const FtAttnArgs& a, const FtNoise& noise, float tau, uintptr_t kf_score, uintptr_t ws, size_t ws_bytes,
                            uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_keyformer_fwd(&a, &noise, tau, ptr<float>(kf_score), ptr<void>(ws), ws_bytes, ptr<void>(stream)));
  }, py::arg("args"), py::arg("noise"), py::arg("tau"), py::arg("kf_score"), py::arg("workspace"), py::arg("workspace_bytes"),
     py::arg("stream") = 0);

  m.def("attn_softcap_fwd", [](const FtAttnArgs& a, float softcap, uintptr_t lse, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_attn_softcap_fwd(&a, softcap, ptr<float>(lse), ptr<void>(stream)));
  }, py::arg("args"), py::arg("softcap"), py::arg("lse") = 0, py::arg("stream") = 0);

  m.def("corm_fwd", [](const FtAttnArgs& a, uintptr_t corm_mask, int64_t mask_row_stride, uintptr_t corm_score, uintptr_t margin,
                       uintptr_t ws, size_t ws_bytes, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_corm_fwd(&a, ptr<const float>(corm_mask), mask_row_stride, ptr<uint8_t>(corm_score), ptr<float>(margin), ptr<void>(ws),
                      ws_bytes, ptr<void>(stream)));
  }, py::arg("args"), py::arg("corm_mask"), py::arg("mask_row_stride"), py::arg("corm_score"), py::arg("margin"), py::arg("workspace"),
     py::arg("workspace_bytes"), py::arg("stream") = 0);

  m.def("avgpool1d", [](uintptr_t src, int64_t rows, int32_t S, int32_t kernel, uintptr_t dst, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_avgpool1d(ptr<const float>(src), rows, S, kernel, ptr<float>(dst), ptr<void>(stream)));
  }, py::arg("src"), py::arg("rows"), py::arg("S"), py::arg("kernel"), py::arg("dst"), py::arg("stream") = 0);

  m.def("linattn_fwd", [](const FtAttnArgs& a, int kind, int normalize_q, int out_dtype, uintptr_t ws, size_t ws_bytes, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_linattn_fwd(&a, kind, normalize_q, out_dtype, ptr<void>(ws), ws_bytes, ptr<void>(stream)));
  }, py::arg("args"), py::arg("kind"), py::arg("normalize_q"), py::arg("out_dtype"), py::arg("workspace"), py::arg("workspace_bytes"),
     py::arg("stream") = 0);

  m.def("linattn_block_workspace_bytes", [](const FtLinBlockArgs& b, int kind) { return ft_linattn_block_workspace_bytes(&b, kind); });

  m.def("linattn_block_fwd", [](const FtLinBlockArgs& b, int kind, int normalize_q, uintptr_t ws, size_t ws_bytes, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_linattn_block_fwd(&b, kind, normalize_q, ptr<void>(ws), ws_bytes, ptr<void>(stream)));
  }, py::arg("args"), py::arg("kind"), py::arg("normalize_q"), py::arg("workspace"), py::arg("workspace_bytes"), py::arg("stream") = 0);

  m.def("topk", [](uintptr_t score, int64_t rows, int32_t S, int32_t k, uintptr_t idx, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_topk(ptr<const float>(score), rows, S, k, ptr<int64_t>(idx), ptr<void>(stream)));
  }, py::arg("score"), py::arg("rows"), py::arg("S"), py::arg("k"), py::arg("idx"), py::arg("stream") = 0);

  m.def("noise_exp_fill", [](uintptr_t dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed, uintptr_t stream) {
    py::gil_scoped_release nogil;
    check(ft_noise_exp_fill(ptr<float>(dst), B, H, Sq, Skv, seed, ptr<void>(stream)));
  }, py::arg("dst"), py::arg("B"), py::arg("H"), py::arg("Sq"), py::arg("Skv"), py::arg("seed"), py::arg("stream") = 0);

  m.def("noise_exp_fill_host", [](uintptr_t dst, int32_t B, int32_t H, int32_t Sq, int32_t Skv, uint64_t seed) {
    py::gil_scoped_release nogil;
    check(ft_noise_exp_fill_host(ptr<float>(dst), B, H, Sq, Skv, seed));
  }, py::arg("dst"), py::arg("B"), py::arg("H"), py::arg("Sq"), py::arg("Skv"), py::arg("seed"));
}

PYBIND11_MODULE(ft_ffi, m) {
  m.doc() = "flashtensor_amd native bindings";
  init_ffi_kernels(m.def_submodule("kernels"));
}
