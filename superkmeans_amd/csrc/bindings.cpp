// pybind11 module `_superkmeans` over the HIP-backed host classes.
//
// Exposes the names and members the reference's module exposes
// (python/bindings/bindings.cpp: SuperKMeansConfig :29-106, SuperKMeansIterationStats :108-156,
// SuperKMeans :158-378, HierarchicalSuperKMeansConfig :380-409,
// HierarchicalSuperKMeansIterationStats :411-431, HierarchicalSuperKMeans :433-670), so the Python
// package on top of it keeps working unchanged.
#include <pybind11/numpy.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <cstring>
#include <string>

#include "superkmeans/hierarchical_superkmeans.h"
#include "superkmeans/superkmeans.h"

namespace py = pybind11;
using skmeans::HierarchicalSuperKMeansConfig;
using skmeans::HierarchicalSuperKMeansIterationStats;
using skmeans::SuperKMeansConfig;
using skmeans::SuperKMeansIterationStats;
using Flat = skmeans::SuperKMeans<skmeans::Quantization::f32, skmeans::DistanceFunction::l2>;
using Hier = skmeans::HierarchicalSuperKMeans<skmeans::Quantization::f32, skmeans::DistanceFunction::l2>;
using f32_array = py::array_t<float>;

namespace {

struct Matrix {
    const float* ptr;
    size_t rows, cols;
};

// Rank and layout rules of the reference's ValidatePyArray (bindings.cpp:11-23).
Matrix as_matrix(const f32_array& arr, const std::string& name) {
    if (arr.ndim() != 2)
        throw std::runtime_error(name + " must be a 2-dimensional array, got " + std::to_string(arr.ndim()));
    if (!(arr.flags() & py::array::c_style)) throw std::runtime_error(name + " must be C-contiguous (row-major)");
    return {arr.data(), static_cast<size_t>(arr.shape(0)), static_cast<size_t>(arr.shape(1))};
}

template <class Model>
f32_array do_train(Model& self, const f32_array& data, const py::object& queries_obj, size_t n_queries) {
    const Matrix x = as_matrix(data, "data");
    const float* q_ptr = nullptr;
    f32_array queries;
    if (!queries_obj.is_none()) {
        queries = queries_obj.cast<f32_array>();
        const Matrix q = as_matrix(queries, "queries");
        if (q.cols != x.cols) throw std::runtime_error("queries must have the same dimensionality as data");
        n_queries = q.rows;
        q_ptr = q.ptr;
    }
    const auto c = self.Train(x.ptr, x.rows, q_ptr, n_queries);
    f32_array out({self.GetNClusters(), x.cols});
    std::memcpy(out.mutable_data(), c.data(), c.size() * sizeof(float));
    return out;
}

template <class Model, class Fn>
py::array_t<uint32_t> do_assign(Model& self, const f32_array& vectors, const f32_array& centroids, Fn fn) {
    const Matrix v = as_matrix(vectors, "vectors"), c = as_matrix(centroids, "centroids");
    if (v.cols != c.cols) throw std::runtime_error("vectors and centroids must have the same dimensionality");
    const auto a = fn(self, v.ptr, c.ptr, v.rows, c.rows);
    py::array_t<uint32_t> out(static_cast<py::ssize_t>(a.size()));
    std::memcpy(out.mutable_data(), a.data(), a.size() * sizeof(uint32_t));
    return out;
}

template <class Model, class PyClass>
void add_model_methods(PyClass& cls) {
    cls.def(
           "train",
           [](Model& self, f32_array data, py::object queries, size_t n_queries) {
               return do_train(self, data, queries, n_queries);
           },
           py::arg("data"), py::arg("queries") = py::none(), py::arg("n_queries") = 0,
           "Run k-means on an (n, d) float32 array; returns the (n_clusters, d) centroids.")
        .def(
            "assign",
            [](Model& self, f32_array vectors, f32_array centroids) {
                return do_assign(self, vectors, centroids, [](Model& m, const float* v, const float* c, size_t nv, size_t nc) {
                    return m.Assign(v, c, nv, nc);
                });
            },
            py::arg("vectors"), py::arg("centroids"), "Exact nearest-centroid index of every vector (uint32).")
        .def(
            "assign_training_points",
            [](Model& self, f32_array vectors, f32_array centroids) {
                return do_assign(self, vectors, centroids, [](Model& m, const float* v, const float* c, size_t nv, size_t nc) {
                    return m.AssignTrainingPoints(v, c, nv, nc);
                });
            },
            py::arg("vectors"), py::arg("centroids"),
            "Pruned assignment of the points used in train(), seeded with the training assignments.")
        .def("get_n_clusters", &Model::GetNClusters)
        .def("is_trained", &Model::IsTrained)
        .def_readonly("iteration_stats", &Model::iteration_stats);
}

} // namespace

PYBIND11_MODULE(_superkmeans, m) {
    m.doc() = "Super K-Means for high-dimensional vectors: HIP backend for AMD MI355X (gfx950)";

    py::class_<SuperKMeansConfig>(m, "SuperKMeansConfig", "Configuration parameters for SuperKMeans clustering.")
        .def(py::init<>())
        .def_readwrite("iters", &SuperKMeansConfig::iters)
        .def_readwrite("sampling_fraction", &SuperKMeansConfig::sampling_fraction)
        .def_readwrite("max_points_per_cluster", &SuperKMeansConfig::max_points_per_cluster)
        .def_readwrite("n_threads", &SuperKMeansConfig::n_threads)
        .def_readwrite("seed", &SuperKMeansConfig::seed)
        .def_readwrite("use_blas_only", &SuperKMeansConfig::use_blas_only)
        .def_readwrite("tol", &SuperKMeansConfig::tol)
        .def_readwrite("recall_tol", &SuperKMeansConfig::recall_tol)
        .def_readwrite("early_termination", &SuperKMeansConfig::early_termination)
        .def_readwrite("sample_queries", &SuperKMeansConfig::sample_queries)
        .def_readwrite("objective_k", &SuperKMeansConfig::objective_k)
        .def_readwrite("verbose", &SuperKMeansConfig::verbose)
        .def_readwrite("angular", &SuperKMeansConfig::angular)
        .def_readwrite("dct_rotation", &SuperKMeansConfig::dct_rotation)
        .def("__repr__", [](const SuperKMeansConfig& c) {
            return "<SuperKMeansConfig: iters=" + std::to_string(c.iters) +
                   ", sampling_fraction=" + std::to_string(c.sampling_fraction) +
                   ", n_threads=" + std::to_string(c.n_threads) + ">";
        });

    py::class_<SuperKMeansIterationStats>(m, "SuperKMeansIterationStats", "Statistics of one k-means iteration.")
        .def(py::init<>())
        .def_readonly("iteration", &SuperKMeansIterationStats::iteration)
        .def_readonly("objective", &SuperKMeansIterationStats::objective)
        .def_readonly("shift", &SuperKMeansIterationStats::shift)
        .def_readonly("split", &SuperKMeansIterationStats::split)
        .def_readonly("recall", &SuperKMeansIterationStats::recall)
        .def_readonly("not_pruned_pct", &SuperKMeansIterationStats::not_pruned_pct)
        .def_readonly("partial_d", &SuperKMeansIterationStats::partial_d)
        .def_readonly("is_gemm_only", &SuperKMeansIterationStats::is_gemm_only)
        .def("__repr__", [](const SuperKMeansIterationStats& s) {
            return "<IterationStats: iter=" + std::to_string(s.iteration) + ", objective=" + std::to_string(s.objective) +
                   ", shift=" + std::to_string(s.shift) + ">";
        });

    py::class_<Flat> flat(m, "SuperKMeans", "SuperKMeans clustering");
    flat.def(py::init<size_t, size_t, const SuperKMeansConfig&>(), py::arg("n_clusters"), py::arg("dimensionality"),
             py::arg("config"))
        .def(py::init<size_t, size_t>(), py::arg("n_clusters"), py::arg("dimensionality"))
        .def("__repr__", [](const Flat& s) {
            return "<SuperKMeans: n_clusters=" + std::to_string(s.GetNClusters()) +
                   ", trained=" + (s.IsTrained() ? "True" : "False") + ">";
        });
    add_model_methods<Flat>(flat);

    py::class_<HierarchicalSuperKMeansConfig, SuperKMeansConfig>(m, "HierarchicalSuperKMeansConfig",
                                                                 "Configuration parameters for HierarchicalSuperKMeans.")
        .def(py::init<>())
        .def_readwrite("iters_mesoclustering", &HierarchicalSuperKMeansConfig::iters_mesoclustering)
        .def_readwrite("iters_fineclustering", &HierarchicalSuperKMeansConfig::iters_fineclustering)
        .def_readwrite("iters_refinement", &HierarchicalSuperKMeansConfig::iters_refinement);

    py::class_<HierarchicalSuperKMeansIterationStats>(m, "HierarchicalSuperKMeansIterationStats",
                                                      "Per-phase iteration statistics of HierarchicalSuperKMeans.")
        .def(py::init<>())
        .def_readonly("mesoclustering_iteration_stats", &HierarchicalSuperKMeansIterationStats::mesoclustering_iteration_stats)
        .def_readonly("fineclustering_iteration_stats", &HierarchicalSuperKMeansIterationStats::fineclustering_iteration_stats)
        .def_readonly("refinement_iteration_stats", &HierarchicalSuperKMeansIterationStats::refinement_iteration_stats);

    py::class_<Hier> hier(m, "HierarchicalSuperKMeans", "Hierarchical SuperKMeans clustering");
    hier.def(py::init<size_t, size_t, const HierarchicalSuperKMeansConfig&>(), py::arg("n_clusters"),
             py::arg("dimensionality"), py::arg("config"))
        .def(py::init<size_t, size_t>(), py::arg("n_clusters"), py::arg("dimensionality"))
        .def_readonly("hierarchical_iteration_stats", &Hier::hierarchical_iteration_stats)
        .def("__repr__", [](const Hier& s) {
            return "<HierarchicalSuperKMeans: n_clusters=" + std::to_string(s.GetNClusters()) +
                   ", trained=" + (s.IsTrained() ? "True" : "False") + ">";
        });
    add_model_methods<Hier>(hier);
}
