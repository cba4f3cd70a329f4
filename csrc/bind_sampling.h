// Bindings shared by the native modules: the on-device sampler (with its decode feedback) and the
// host-mapped token ring. Device pointers and streams cross as integers, as in bindings.cpp.
#pragma once
#include <pybind11/pybind11.h>

#include <cstring>
#include <stdexcept>

#include "kernels/ops.h"

namespace omx {

inline void bind_sampling(pybind11::module_& m) {
  namespace py = pybind11;
  m.def("host_alloc_mapped", [](size_t bytes) {
    void* h = nullptr;
    void* d = nullptr;
    if (hipHostMalloc(&h, bytes, hipHostMallocMapped) != hipSuccess || !h)
      throw std::runtime_error("hipHostMalloc(mapped) failed");
    if (hipHostGetDevicePointer(&d, h, 0) != hipSuccess || !d) {
      (void)hipHostFree(h);
      throw std::runtime_error("hipHostGetDevicePointer failed");
    }
    std::memset(h, 0, bytes);
    return py::make_tuple((uintptr_t)h, (uintptr_t)d);
  });
  m.def("host_free_mapped", [](uintptr_t h) {
    if (h) (void)hipHostFree((void*)h);
  });
  m.def("sample", [](py::dict d, uintptr_t stream) {
    SampleParams P{};
    P.logits = reinterpret_cast<const float*>(d["logits"].cast<uintptr_t>());
    P.B = d["B"].cast<int>();
    P.V = d["V"].cast<int>();
    P.ld = d["ld"].cast<int>();
    P.temperature = reinterpret_cast<const float*>(d["temperature"].cast<uintptr_t>());
    P.top_k = reinterpret_cast<const int*>(d["top_k"].cast<uintptr_t>());
    P.top_p = reinterpret_cast<const float*>(d["top_p"].cast<uintptr_t>());
    P.min_p = reinterpret_cast<const float*>(d["min_p"].cast<uintptr_t>());
    P.repeat_penalty = reinterpret_cast<const float*>(d["repeat_penalty"].cast<uintptr_t>());
    P.presence_penalty = reinterpret_cast<const float*>(d["presence_penalty"].cast<uintptr_t>());
    P.frequency_penalty = reinterpret_cast<const float*>(d["frequency_penalty"].cast<uintptr_t>());
    P.history = reinterpret_cast<int*>(d["history"].cast<uintptr_t>());
    P.hist_count = reinterpret_cast<int*>(d["hist_count"].cast<uintptr_t>());
    P.hist_cap = d["hist_cap"].cast<int>();
    P.repeat_last_n = reinterpret_cast<const int*>(d["repeat_last_n"].cast<uintptr_t>());
    P.seed = reinterpret_cast<const unsigned long long*>(d["seed"].cast<uintptr_t>());
    P.step = reinterpret_cast<int*>(d["step"].cast<uintptr_t>());
    P.out = reinterpret_cast<int*>(d["out"].cast<uintptr_t>());
    P.out_logprob = reinterpret_cast<float*>(d.contains("out_logprob") ? d["out_logprob"].cast<uintptr_t>() : 0);
    P.ws = reinterpret_cast<float*>(d.contains("ws") ? d["ws"].cast<uintptr_t>() : 0);
    P.counters = reinterpret_cast<int*>(d.contains("counters") ? d["counters"].cast<uintptr_t>() : 0);
    P.err = reinterpret_cast<int*>(d.contains("err") ? d["err"].cast<uintptr_t>() : 0);
    if (d.contains("fb_step")) {
      P.fb_step = reinterpret_cast<int*>(d["fb_step"].cast<uintptr_t>());
      P.fb_ld = d["fb_ld"].cast<int>();
      P.fb_block_table = reinterpret_cast<const int*>(d["fb_block_table"].cast<uintptr_t>());
      P.fb_max_blocks = d["fb_max_blocks"].cast<int>();
      P.fb_bs = d["fb_bs"].cast<int>();
      P.fb_host_ring = reinterpret_cast<int*>(d.contains("fb_host_ring") ? d["fb_host_ring"].cast<uintptr_t>() : 0);
      P.fb_ring = d.contains("fb_ring") ? d["fb_ring"].cast<int>() : 0;
      P.fb_sysfence = d.contains("fb_sysfence") ? d["fb_sysfence"].cast<int>() : 1;
      if (P.B > P.fb_ld || P.fb_bs <= 0 || P.fb_max_blocks <= 0) throw std::runtime_error("sample: bad feedback args");
      if (P.fb_host_ring && P.fb_ring <= 0) throw std::runtime_error("sample: bad feedback ring");
    }
    sample(P, reinterpret_cast<hipStream_t>(stream));
  });
}

}  // namespace omx
