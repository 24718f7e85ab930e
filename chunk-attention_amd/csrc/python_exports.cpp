// Python module chunk_attn_c: the binding surface of the reference's module of the same name
// (cpp/chunk_attn/python_exports.cpp:11-87 there) over the MI355X implementation.
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>
#include <torch/extension.h>

#include "attention.h"

namespace py = pybind11;
using GPT::Attention;
using GPT::Chunk;

PYBIND11_MODULE(chunk_attn_c, m) {
    m.doc() = "ChunkAttention decode path for MI355X (prefix-tree KV cache + HIP kernels)";

    py::class_<std::future<int>, std::shared_ptr<std::future<int>>>(m, "IntFuture")
      .def(py::init<>())
      .def("get", &std::future<int>::get);

    py::class_<Chunk>(m, "Chunk")
      .def_readonly("children", &Chunk::children, py::return_value_policy::reference)
      .def_readonly("tokens", &Chunk::tokens)
      .def_property_readonly("capacity", &Chunk::capacity)
      .def_readonly("n_seqs", &Chunk::n_seqs)
      .def_property_readonly("n_tokens", &Chunk::n_tokens)
      .def_property_readonly("slot", &Chunk::slot);

    py::class_<Attention, std::shared_ptr<Attention>>(m, "Attention")
      .def(py::init([](int n_heads, int d_head, int chunk_size, int memory_mb, bool share_prefix,
                       int tpp_threshold, py::object dtype, py::object device) {
               torch::Dtype dtype_c = torch::get_default_dtype_as_scalartype();
               if (!dtype.is_none()) dtype_c = torch::python::detail::py_object_to_dtype(dtype);
               // device None = wherever new tensors go by default (torch.set_default_device)
               torch::Device device_c = torch::empty({ 1 }).device();
               if (!device.is_none()) device_c = torch::python::detail::py_object_to_device(device);
               return std::make_shared<Attention>(n_heads, d_head, chunk_size, memory_mb, share_prefix,
                                                  tpp_threshold, dtype_c, device_c);
           }),
           py::arg("n_heads") = 12, py::arg("d_head") = 64, py::arg("chunk_size") = 64,
           py::arg("memory_mb") = 1024, py::arg("share_prefix") = true, py::arg("tpp_threshold") = 1,
           py::arg("dtype") = py::none(), py::arg("device") = py::none())
      .def(py::init<Attention&>())
      .def("forward", &Attention::forward, py::arg("q"), py::arg("partition") = 0)
      .def("add_seq", &Attention::add_seq, py::arg("tokens"), py::arg("k"), py::arg("v"))
      .def("add_seq_async", &Attention::add_seq_async, py::arg("tokens"), py::arg("k"), py::arg("v"))
      .def("append_token", &Attention::append_token, py::arg("tokens"), py::arg("k"), py::arg("v"),
           py::arg("fused") = true, py::return_value_policy::reference)
      .def("append_token_rotary", &Attention::append_token_rotary, py::arg("tokens"), py::arg("q"), py::arg("k"),
           py::arg("v"), py::arg("cos_sin_cache"), py::arg("is_neox") = true, py::arg("positions") = py::none(),
           py::return_value_policy::reference)
      .def("decode_step", &Attention::decode_step, py::arg("tokens"), py::arg("q"), py::arg("k"), py::arg("v"))
      .def("refresh_kernel_context", &Attention::refresh_kernel_context, py::arg("force") = false)
      .def("reserve", &Attention::reserve, py::return_value_policy::reference)
      .def("duplicate", &Attention::duplicate, py::arg("seq_idx"), py::arg("copies"))
      .def("append_completion", &Attention::append_completion, py::arg("seq_idx"), py::arg("tokens"),
           py::arg("k"), py::arg("v"))
      .def("remove_seq", &Attention::remove_seq, py::arg("seq_idx"))
      .def("clear", &Attention::clear)
      .def("get_trie", &Attention::get_trie, py::return_value_policy::reference)
      .def_property_readonly("tails", &Attention::tails, py::return_value_policy::reference)
      .def("print", &Attention::print, py::arg("root") = nullptr, py::arg("level") = 0)
      .def("peak_memory_allocated", &Attention::peak_memory_allocated)
      .def("get_chunks",
           [](Attention& a) {
               std::vector<std::tuple<Chunk*, int, int>> out;
               for (const auto& r : a.get_chunks()) out.emplace_back(r.chunk, r.seq_idx_begin, r.seq_idx_end);
               return out;
           },
           py::return_value_policy::reference)
      .def("key", &Attention::key, py::arg("chunk"))
      .def("value", &Attention::value, py::arg("chunk"));

    // the reference's chunk_attn.ops module (cpp/chunk_attn/python_exports_ops.cpp:11-19), the part the
    // decode path's callers use (all three of its operators)
    py::module ops = m.def_submodule("ops", "operators used around the attention call");
    ops.def("rotary_embedding", &GPT::rotary_embedding, py::arg("positions"), py::arg("query"), py::arg("key"),
            py::arg("head_size"), py::arg("cos_sin_cache"), py::arg("is_neox"),
            "Apply GPT-NeoX or GPT-J style rotary embedding to query and key");
    ops.def("rms_norm", &GPT::rms_norm, py::arg("out"), py::arg("input"), py::arg("weight"), py::arg("epsilon"),
            "Apply Root Mean Square (RMS) Normalization to the input tensor.");
    ops.def("fused_add_rms_norm", &GPT::fused_add_rms_norm, py::arg("input"), py::arg("residual"),
            py::arg("weight"), py::arg("epsilon"), "In-place fused Add and RMS Normalization");
}
