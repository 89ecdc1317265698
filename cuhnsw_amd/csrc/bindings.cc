// pybind11 module cuhnsw_bind: class CuHNSWBind with the method names, argument
// names and error behaviour of the reference's binding (cuhnsw/bindings.cc:18-94 in
// js1010/cuhnsw), implemented as a thin shim over the C ABI in include/cuhnsw_amd.h.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>

#include <stdexcept>
#include <string>

#include "cuhnsw_amd.h"

namespace py = pybind11;

typedef py::array_t<float, py::array::c_style | py::array::forcecast> float_array;
typedef py::array_t<int, py::array::c_style | py::array::forcecast> int_array;

class CuHNSWBind {
 public:
  CuHNSWBind() {
    if (cuhnsw_create(&obj_) != 0) throw std::runtime_error(std::string("cannot create engine: ") + cuhnsw_last_error(nullptr));
  }
  ~CuHNSWBind() { cuhnsw_destroy(obj_); }
  CuHNSWBind(const CuHNSWBind&) = delete;
  CuHNSWBind& operator=(const CuHNSWBind&) = delete;

  bool Init(std::string opt_path) {
    int rc = cuhnsw_init(obj_, opt_path.c_str());
    if (rc == 2) throw std::runtime_error(cuhnsw_last_error(obj_));  // invalid dist type
    return rc == 0;
  }
  void SetData(py::object& input) {
    float_array array(input);
    auto buffer = array.request();
    if (buffer.ndim != 2) throw std::runtime_error("data must be 2d array");
    Check(cuhnsw_set_data(obj_, array.data(0), (int)buffer.shape[0], (int)buffer.shape[1]));
  }
  void BuildGraph() {
    py::gil_scoped_release release;
    Check(cuhnsw_build_graph(obj_));
  }
  void SetRandomLevels(py::object& input) {
    int_array array(input);
    auto buffer = array.request();
    if (buffer.ndim != 1) throw std::runtime_error("levels must be 1d array");
    Check(cuhnsw_set_random_levels(obj_, array.data(0), (int)buffer.shape[0]));
  }
  void SaveIndex(std::string fpath) { Check(cuhnsw_save_index(obj_, fpath.c_str())); }
  void LoadIndex(std::string fpath) { Check(cuhnsw_load_index(obj_, fpath.c_str())); }
  void SearchGraph(py::object& qdata, int topk, int ef_search, py::object& nns, py::object& distances,
                   py::object& found_cnt) {
    float_array _qdata(qdata);
    int_array _nns(nns);
    float_array _distances(distances);
    int_array _found_cnt(found_cnt);
    auto buffer = _qdata.request();
    if (buffer.ndim != 1 && buffer.ndim != 2) throw std::runtime_error("data array must be 1d / 2d shape");
    int num_queries = buffer.ndim == 1 ? 1 : (int)buffer.shape[0];
    int dims = (int)buffer.shape[buffer.ndim - 1];
    if (dims != cuhnsw_num_dims(obj_)) throw std::runtime_error("query dimension differs from the index dimension");
    if ((long long)_nns.size() < (long long)num_queries * topk || (long long)_distances.size() < (long long)num_queries * topk ||
        (long long)_found_cnt.size() < num_queries)
      throw std::runtime_error("output arrays are too small");
    const float* q = _qdata.data(0);
    int* out_nns = _nns.mutable_data(0);
    float* out_distances = _distances.mutable_data(0);
    int* out_found = _found_cnt.mutable_data(0);
    int rc;
    {
      // plain pointers from here on: other Python threads may run while the GPU searches
      py::gil_scoped_release release;
      rc = cuhnsw_search_knn(obj_, q, num_queries, topk, ef_search, out_nns, out_distances, out_found);
    }
    Check(rc);
  }
  // not in the reference: engine facts and tuning knobs
  int NumData() const { return cuhnsw_num_data(obj_); }
  int NumDims() const { return cuhnsw_num_dims(obj_); }
  int MaxLevel() const { return cuhnsw_max_level(obj_); }
  int EnterPoint() const { return cuhnsw_enter_point(obj_); }
  double LastBuildSeconds() const { return cuhnsw_last_build_seconds(obj_); }
  void SetTunable(std::string name, double value) {
    const int rc = cuhnsw_set_tunable(obj_, name.c_str(), value);
    if (rc == -2) throw std::runtime_error("tunable " + name + " has to be set before set_data / load_index");
    if (rc != 0) throw std::runtime_error("unknown tunable " + name);
  }

 private:
  void Check(int rc) {
    if (rc != 0) throw std::runtime_error(cuhnsw_last_error(obj_));
  }
  cuhnsw_engine* obj_ = nullptr;
};

PYBIND11_MODULE(cuhnsw_bind, m) {
  m.def("has_device", []() { return cuhnsw_has_device() != 0; });
  py::class_<CuHNSWBind>(m, "CuHNSWBind")
      .def(py::init())
      .def("init", &CuHNSWBind::Init, py::arg("opt_path"))
      .def("set_data", &CuHNSWBind::SetData, py::arg("data"))
      .def("build_graph", &CuHNSWBind::BuildGraph)
      .def("set_random_levels", &CuHNSWBind::SetRandomLevels, py::arg("levels"))
      .def("save_index", &CuHNSWBind::SaveIndex, py::arg("fpath"))
      .def("load_index", &CuHNSWBind::LoadIndex, py::arg("fpath"))
      .def("search_knn", &CuHNSWBind::SearchGraph, py::arg("qdata"), py::arg("topk"), py::arg("ef_search"),
           py::arg("nns"), py::arg("distances"), py::arg("found"))
      .def("num_data", &CuHNSWBind::NumData)
      .def("num_dims", &CuHNSWBind::NumDims)
      .def("max_level", &CuHNSWBind::MaxLevel)
      .def("enter_point", &CuHNSWBind::EnterPoint)
      .def("last_build_seconds", &CuHNSWBind::LastBuildSeconds)
      .def("set_tunable", &CuHNSWBind::SetTunable, py::arg("name"), py::arg("value"))
      .def("__repr__", [](const CuHNSWBind&) { return "<CuHNSWBind>"; });
}
