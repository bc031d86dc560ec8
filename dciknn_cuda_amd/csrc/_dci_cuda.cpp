// Torch C++ extension `_dci_cuda`: the seven functions the reference's Python
// layer imports (dciknn_cuda/core.py:19, bound at src/dci_cuda.cpp:175-183), here
// as a thin layer over the C-ABI of libdci_hip.so.  Tensors stay torch's, work
// goes to torch's current HIP stream, errors become Python exceptions.
//
// Unlike src/dci_cuda.cpp the capsule owns a small host struct, so an explicit
// _dci_free followed by the capsule's destructor releases the index once; query
// results are ordinary torch tensors (the reference leaks two cudaMalloc blocks
// per query, :100-113); no Python object is touched from another thread.
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <torch/extension.h>

#include <algorithm>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/dci_hip.h"

namespace py = pybind11;

namespace {

struct Holder {
    dcih_index* h = nullptr;
    int device = 0;
};

constexpr const char* kCapsuleName = "py_dci_inst";   // name kept from src/dci_cuda.cpp:64

void check(int rc) {
    if (rc < 0) throw std::runtime_error(std::string("libdci_hip: ") + dcih_last_error());
}

Holder* holder(const py::handle& capsule) {
    auto* p = static_cast<Holder*>(PyCapsule_GetPointer(capsule.ptr(), kCapsuleName));
    if (!p) throw py::error_already_set();
    return p;
}

dcih_index* index_of(const py::handle& capsule) {
    Holder* p = holder(capsule);
    if (!p->h) throw std::runtime_error("this DCI instance has been freed");
    return p->h;
}

void* stream_of(const torch::Tensor& t) {
    return (void*)c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

void capsule_destructor(PyObject* capsule) {
    auto* p = static_cast<Holder*>(PyCapsule_GetPointer(capsule, kCapsuleName));
    if (!p) return;
    if (p->h) dcih_free(p->h);
    delete p;
}

void require_f32_device(const torch::Tensor& t, const char* what) {
    TORCH_CHECK(t.is_cuda(), what, " must live on the GPU");
    TORCH_CHECK(t.scalar_type() == torch::kFloat32, what, " must be float32");
    TORCH_CHECK(t.is_contiguous(), what, " must be contiguous");
}

// src/dci_cuda.cpp:54-66 (py_dci_new); `seed` is an addition (directions are drawn on the host).
py::object dci_new(int dim, int num_comp_indices, int num_simp_indices, int device_id,
                   unsigned long long seed) {
    auto* p = new Holder();
    p->device = device_id;
    const int rc = dcih_create(dim, num_comp_indices, num_simp_indices, device_id, seed, &p->h);
    if (rc < 0) {
        delete p;
        check(rc);
    }
    return py::reinterpret_steal<py::object>(PyCapsule_New(p, kCapsuleName, capsule_destructor));
}

// src/dci_cuda.cpp:68-82 (py_dci_add).  The index borrows the tensor's memory; the
// Python layer keeps the tensor alive (core.py:75).
void dci_add(py::handle capsule, int dim, int64_t num_points, torch::Tensor data,
             int block_size, int thread_size) {
    require_f32_device(data, "data");
    TORCH_CHECK(data.numel() == num_points * (int64_t)dim, "data has the wrong number of elements");
    c10::DeviceGuard guard(data.device());
    check(dcih_add(index_of(capsule), dim, num_points, data.data_ptr<float>(), block_size,
                   thread_size, stream_of(data)));
}

// src/dci_cuda.cpp:84-118 (py_dci_query): flat float32 tensor, first half the ids
// (as floats, like the reference), second half the distances.  Blind: per query
// min(max_num_candidates, num_outer_iterations) candidate ids (the size
// src/dci_cuda_kernel.cu:775-783 asks for; the reference's own buffer at :99 is
// too small for it), second half the steps at which they were promoted.
torch::Tensor dci_query(py::handle capsule, int dim, int num_queries, torch::Tensor query,
                        int num_neighbours, bool blind, int num_outer_iterations,
                        int max_num_candidates, int block_size, int thread_size) {
    require_f32_device(query, "query");
    TORCH_CHECK(query.numel() == (int64_t)num_queries * dim, "query has the wrong number of elements");
    c10::DeviceGuard guard(query.device());
    const int64_t per_query = blind ? std::min(max_num_candidates, num_outer_iterations) : num_neighbours;
    TORCH_CHECK(per_query > 0, "nothing to return per query");
    const int64_t cells = (int64_t)num_queries * per_query;
    auto ids = torch::empty({cells}, query.options().dtype(torch::kInt32));
    auto dists = torch::empty({cells}, query.options());
    check(dcih_query(index_of(capsule), dim, num_queries, query.data_ptr<float>(), num_neighbours,
                     blind ? 1 : 0, num_outer_iterations, max_num_candidates, block_size,
                     thread_size, ids.data_ptr<int32_t>(), dists.data_ptr<float>(), nullptr,
                     stream_of(query)));
    return torch::cat({ids.to(torch::kFloat32), dists}, 0);
}

// src/dci_cuda.cpp:120-134 (py_dci_multi_query).  One GPU per process here, so the
// lists hold one entry; the reference's std::async fan-out has nothing to fan out to.
std::vector<torch::Tensor> dci_multi_query(std::vector<py::handle> capsules, int dim, int num_queries,
                                           std::vector<torch::Tensor> queries, int num_neighbours,
                                           bool blind, int num_outer_iterations,
                                           int max_num_candidates, int block_size, int thread_size) {
    TORCH_CHECK(capsules.size() == queries.size(), "one query tensor per DCI instance");
    TORCH_CHECK(capsules.size() == 1, "this build runs on one GPU");
    return {dci_query(capsules[0], dim, num_queries, queries[0], num_neighbours, blind,
                      num_outer_iterations, max_num_candidates, block_size, thread_size)};
}

void dci_clear(py::handle capsule) { check(dcih_clear(index_of(capsule))); }   // :136-147
void dci_reset(py::handle capsule) { check(dcih_reset(index_of(capsule))); }   // :149-160

void dci_free(py::handle capsule) {                                            // :162-173
    Holder* p = holder(capsule);
    if (p->h) {
        dcih_free(p->h);
        p->h = nullptr;
    }
}

// Address of the C-ABI handle, for the entry points the reference has no function for
// (directions, counters, options): those are called through the C-ABI directly.
uintptr_t dci_handle(py::handle capsule) { return reinterpret_cast<uintptr_t>(holder(capsule)->h); }

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("_dci_new", &dci_new, "Create new DCI instance. (HIP)", py::arg("dim"),
          py::arg("num_comp_indices"), py::arg("num_simp_indices"), py::arg("device_id"),
          py::arg("seed") = 0ull);
    m.def("_dci_add", &dci_add, "Add data. (HIP)");
    m.def("_dci_query", &dci_query, "Search for nearest neighbours. (HIP)");
    m.def("_dci_clear", &dci_clear, "Clear DCI. (HIP)");
    m.def("_dci_reset", &dci_reset, "Reset DCI. (HIP)");
    m.def("_dci_free", &dci_free, "Free DCI. (HIP)");
    m.def("_dci_multi_query", &dci_multi_query, "Search on several DCI instances (one GPU: one instance). (HIP)");
    m.def("_dci_handle", &dci_handle, "Address of the libdci_hip handle.");
}
