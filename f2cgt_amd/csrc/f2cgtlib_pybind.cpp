// Python module `F2CGTLib`: the operator surface of the reference's pybind module
// (src/pybind.cu:7-48: same function names, keyword names, argument order, tensor
// layouts and return types) on top of the C ABI of libf2cgt_hip.so.
//
// This file holds no device code.  It validates arguments (TORCH_CHECK -> RuntimeError
// where the reference aborts or reads out of bounds), allocates the result with torch,
// picks up torch's current HIP stream and forwards raw pointers.
#include <pybind11/pybind11.h>
#include <torch/extension.h>

#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <string>

#include "../../include/f2cgt.h"

namespace py = pybind11;

namespace {

void* current_stream() { return static_cast<void*>(c10::hip::getCurrentHIPStream().stream()); }

void check_rc(int rc, const char* op) {
  TORCH_CHECK(rc == 0, op, " failed (", rc, "): ", f2cgt_last_error());
}

torch::Tensor dev_contig(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined(), name, " is undefined");
  TORCH_CHECK(t.device().is_cuda(), name, " must be a GPU tensor");
  return t.contiguous();
}

int dtype_tag(const torch::Tensor& t, const char* name) {
  switch (t.scalar_type()) {
    case torch::kUInt8: return F2CGT_DT_U8;
    case torch::kInt8: return F2CGT_DT_I8;
    case torch::kInt16: return F2CGT_DT_I16;
    case torch::kInt32: return F2CGT_DT_I32;
    case torch::kInt64: return F2CGT_DT_I64;
    case torch::kFloat16: return F2CGT_DT_F16;
    case torch::kFloat32: return F2CGT_DT_F32;
    case torch::kFloat64: return F2CGT_DT_F64;
    default: TORCH_CHECK(false, name, " has an unsupported dtype ", t.scalar_type());
  }
  return -1;
}

// CSC index tensors: int32/int64 go straight through; the narrower integer types the
// reference also dispatches on (src/common.h:33-53) are widened to int32 first.
struct Graph {
  torch::Tensor indptr, indices;
  int tag;
  int64_t rows, edges;
};

Graph graph_of(const torch::Tensor& indptr_in, const torch::Tensor& indices_in) {
  Graph g;
  g.indptr = dev_contig(indptr_in, "indptr");
  g.indices = dev_contig(indices_in, "indices");
  TORCH_CHECK(g.indptr.dim() == 1 && g.indptr.numel() >= 1, "indptr must be 1-D with at least one entry");
  TORCH_CHECK(g.indices.dim() == 1, "indices must be 1-D");
  TORCH_CHECK(g.indptr.scalar_type() == g.indices.scalar_type(),
              "indptr and indices must share one integer dtype");
  auto st = g.indptr.scalar_type();
  TORCH_CHECK(st == torch::kInt64 || st == torch::kInt32 || st == torch::kInt16 || st == torch::kInt8 ||
                  st == torch::kUInt8,
              "indptr/indices must be int64, int32, int16, int8 or uint8");
  if (st != torch::kInt64 && st != torch::kInt32) {
    g.indptr = g.indptr.to(torch::kInt32);
    g.indices = g.indices.to(torch::kInt32);
  }
  g.tag = g.indptr.scalar_type() == torch::kInt64 ? F2CGT_DT_I64 : F2CGT_DT_I32;
  g.rows = g.indptr.numel() - 1;
  g.edges = g.indices.numel();
  return g;
}

torch::Tensor empty_f32(std::initializer_list<int64_t> shape, const torch::Tensor& like) {
  return torch::empty(shape, torch::TensorOptions().dtype(torch::kFloat32).device(like.device()));
}

int metric_tag(const std::string& metric) {
  // "cosine" selects cosine; every other string selects squared L2 (src/kmeans.cu:108-112).
  return metric == "cosine" ? F2CGT_METRIC_COSINE : F2CGT_METRIC_L2;
}

// ---- reference operator surface -----------------------------------------------------

torch::Tensor packbits(torch::Tensor unpack, int64_t target_bits) {
  unpack = dev_contig(unpack, "unpack");
  TORCH_CHECK(unpack.dim() == 2, "unpack must be 2-D");
  TORCH_CHECK(unpack.scalar_type() == torch::kUInt8 || unpack.scalar_type() == torch::kInt8,
              "unpack must be uint8");
  TORCH_CHECK(target_bits == 1 || target_bits == 2 || target_bits == 4,
              "packbits: target_bits must be 1, 2 or 4");
  c10::DeviceGuard guard(unpack.device());
  const int64_t per = 8 / target_bits;
  const int64_t pack_dim = (unpack.size(1) + per - 1) / per;
  auto pack = torch::empty({unpack.size(0), pack_dim},
                           torch::TensorOptions().dtype(torch::kUInt8).device(unpack.device()));
  check_rc(f2cgt_packbits(static_cast<const uint8_t*>(unpack.data_ptr()),
                          static_cast<uint8_t*>(pack.data_ptr()), unpack.size(0), unpack.size(1),
                          (int)target_bits, current_stream()),
           "packbits");
  return pack;
}

torch::Tensor unpackbits(torch::Tensor pack, int64_t target_bits, int64_t unpack_dim) {
  pack = dev_contig(pack, "pack");
  TORCH_CHECK(pack.dim() == 2, "pack must be 2-D");
  TORCH_CHECK(pack.scalar_type() == torch::kUInt8 || pack.scalar_type() == torch::kInt8,
              "pack must be uint8");
  TORCH_CHECK(target_bits == 1 || target_bits == 2 || target_bits == 4,
              "unpackbits: target_bits must be 1, 2 or 4");
  TORCH_CHECK(unpack_dim >= 0 && unpack_dim <= pack.size(1) * (8 / target_bits),
              "unpackbits: unpack_dim does not fit the packed row");
  c10::DeviceGuard guard(pack.device());
  auto unpack = torch::empty({pack.size(0), unpack_dim},
                             torch::TensorOptions().dtype(torch::kUInt8).device(pack.device()));
  check_rc(f2cgt_unpackbits(static_cast<const uint8_t*>(pack.data_ptr()),
                            static_cast<uint8_t*>(unpack.data_ptr()), pack.size(0), pack.size(1),
                            unpack_dim, (int)target_bits, current_stream()),
           "unpackbits");
  return unpack;
}

torch::Tensor sq_codebooks_checked(torch::Tensor codebooks) {
  codebooks = dev_contig(codebooks, "codebooks");
  TORCH_CHECK(codebooks.scalar_type() == torch::kFloat32, "codebooks must be float32");
  TORCH_CHECK(codebooks.dim() == 2 && codebooks.size(1) == 5 && codebooks.size(0) >= 1,
              "SQ codebooks must be [n_codebooks, 5] = fmin,fmax,emin,emax,mean");
  return codebooks;
}

torch::Tensor sq_compress(torch::Tensor src, torch::Tensor codebooks, int64_t target_bits,
                          int64_t column_slice) {
  src = dev_contig(src, "src");
  TORCH_CHECK(src.dim() == 2 && src.scalar_type() == torch::kFloat32, "src must be float32 [rows, feat_dim]");
  codebooks = sq_codebooks_checked(codebooks);
  c10::DeviceGuard guard(src.device());
  auto out = torch::empty_like(src);
  check_rc(f2cgt_sq_compress(src.data_ptr<float>(), out.data_ptr<float>(), codebooks.data_ptr<float>(),
                             src.size(0), src.size(1), codebooks.size(0), (int)target_bits, column_slice,
                             current_stream()),
           "sq_compress");
  return out;
}

// Extension: the storage tensor in one pass (= sq_compress -> cast -> packbits of the callers).
torch::Tensor sq_encode(torch::Tensor src, torch::Tensor codebooks, int64_t target_bits, int64_t column_slice) {
  src = dev_contig(src, "src");
  TORCH_CHECK(src.dim() == 2 && src.scalar_type() == torch::kFloat32, "src must be float32 [rows, feat_dim]");
  TORCH_CHECK(target_bits == 1 || target_bits == 2 || target_bits == 4 || target_bits == 8 || target_bits == 16,
              "target_bits must be 1, 2, 4, 8 or 16");
  codebooks = sq_codebooks_checked(codebooks);
  c10::DeviceGuard guard(src.device());
  const int64_t d = src.size(1);
  auto out = target_bits < 8
                 ? torch::empty({src.size(0), (d * target_bits + 7) / 8}, src.options().dtype(torch::kInt8))
                 : torch::empty({src.size(0), d}, src.options().dtype(target_bits == 8 ? torch::kInt8 : torch::kInt16));
  check_rc(f2cgt_sq_encode(src.data_ptr<float>(), out.data_ptr(), codebooks.data_ptr<float>(), src.size(0), d,
                           codebooks.size(0), (int)target_bits, column_slice, current_stream()),
           "sq_encode");
  return out;
}

torch::Tensor sq_decompress(torch::Tensor compress_data, torch::Tensor codebooks, int64_t target_bits,
                            int64_t column_slice, int64_t feat_dim) {
  compress_data = dev_contig(compress_data, "compress_data");
  TORCH_CHECK(compress_data.dim() == 2, "compress_data must be 2-D");
  codebooks = sq_codebooks_checked(codebooks);
  c10::DeviceGuard guard(compress_data.device());
  auto out = empty_f32({compress_data.size(0), feat_dim}, compress_data);
  check_rc(f2cgt_sq_decompress(compress_data.data_ptr(), dtype_tag(compress_data, "compress_data"),
                               out.data_ptr<float>(), codebooks.data_ptr<float>(), compress_data.size(0),
                               compress_data.size(1), feat_dim, codebooks.size(0), (int)target_bits,
                               column_slice, current_stream()),
           "sq_decompress");
  return out;
}

torch::Tensor vq_decompress(torch::Tensor index_tensor, torch::Tensor codebooks, int64_t feat_dim) {
  index_tensor = dev_contig(index_tensor, "index_tensor");
  codebooks = dev_contig(codebooks, "codebooks");
  TORCH_CHECK(index_tensor.dim() == 2, "index_tensor must be [rows, n_codebooks]");
  TORCH_CHECK(codebooks.dim() == 3, "VQ codebooks must be [n_codebooks, K, width]");
  TORCH_CHECK(index_tensor.size(1) == codebooks.size(0), "index_tensor has ", index_tensor.size(1),
              " columns but there are ", codebooks.size(0), " codebooks");
  c10::DeviceGuard guard(index_tensor.device());
  auto out = empty_f32({index_tensor.size(0), feat_dim}, index_tensor);
  check_rc(f2cgt_vq_decompress(index_tensor.data_ptr(), dtype_tag(index_tensor, "index_tensor"),
                               codebooks.data_ptr(), dtype_tag(codebooks, "codebooks"),
                               out.data_ptr<float>(), index_tensor.size(0), feat_dim, codebooks.size(0),
                               codebooks.size(1), codebooks.size(2), current_stream()),
           "vq_decompress");
  return out;
}

torch::Tensor spmm_csr(torch::Tensor feat, torch::Tensor indptr, torch::Tensor indices) {
  feat = dev_contig(feat, "feat");
  TORCH_CHECK(feat.dim() == 2, "feat must be 2-D");
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(feat.device());
  auto out = torch::empty({g.rows, feat.size(1)}, feat.options());
  check_rc(f2cgt_spmm_csr(feat.data_ptr(), dtype_tag(feat, "feat"), out.data_ptr(), g.indptr.data_ptr(),
                          g.indices.data_ptr(), g.tag, g.rows, g.edges, feat.size(0), feat.size(1),
                          current_stream()),
           "spmm_csr");
  return out;
}

torch::Tensor vq_decompress_spmm_csr(torch::Tensor compress_feat, torch::Tensor codebooks,
                                     torch::Tensor indptr, torch::Tensor indices, int64_t feat_dim) {
  compress_feat = dev_contig(compress_feat, "compress_feat");
  codebooks = dev_contig(codebooks, "codebooks");
  TORCH_CHECK(compress_feat.dim() == 2, "compress_feat must be [rows, n_codebooks]");
  TORCH_CHECK(codebooks.dim() == 3 && codebooks.scalar_type() == torch::kFloat32,
              "VQ codebooks must be float32 [n_codebooks, K, width]");
  TORCH_CHECK(compress_feat.size(1) == codebooks.size(0), "compress_feat has ", compress_feat.size(1),
              " columns but there are ", codebooks.size(0), " codebooks");
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(compress_feat.device());
  auto out = empty_f32({g.rows, feat_dim}, compress_feat);
  check_rc(f2cgt_vq_decompress_spmm_csr(compress_feat.data_ptr(), dtype_tag(compress_feat, "compress_feat"),
                                        codebooks.data_ptr<float>(), g.indptr.data_ptr(),
                                        g.indices.data_ptr(), g.tag, out.data_ptr<float>(), g.rows, g.edges,
                                        compress_feat.size(0), feat_dim, codebooks.size(0),
                                        codebooks.size(1), codebooks.size(2), current_stream()),
           "vq_decompress_spmm_csr");
  return out;
}

torch::Tensor sq_decompress_spmm_csr(torch::Tensor compress_feat, torch::Tensor codebooks,
                                     torch::Tensor indptr, torch::Tensor indices, int64_t target_bit,
                                     int64_t column_slice, int64_t feat_dim) {
  compress_feat = dev_contig(compress_feat, "compress_feat");
  TORCH_CHECK(compress_feat.dim() == 2, "compress_feat must be 2-D");
  codebooks = sq_codebooks_checked(codebooks);
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(compress_feat.device());
  auto out = empty_f32({g.rows, feat_dim}, compress_feat);
  check_rc(f2cgt_sq_decompress_spmm_csr(compress_feat.data_ptr(), dtype_tag(compress_feat, "compress_feat"),
                                        codebooks.data_ptr<float>(), g.indptr.data_ptr(),
                                        g.indices.data_ptr(), g.tag, out.data_ptr<float>(), g.rows, g.edges,
                                        compress_feat.size(0), compress_feat.size(1), feat_dim,
                                        codebooks.size(0), (int)target_bit, column_slice, current_stream()),
           "sq_decompress_spmm_csr");
  return out;
}

torch::Tensor kmeans_predict_impl(torch::Tensor x, torch::Tensor centers, const std::string& metric,
                                  bool as_u8) {
  x = dev_contig(x, "data");
  centers = dev_contig(centers, "centers");
  TORCH_CHECK(x.dim() == 2 && centers.dim() == 2 && x.size(1) == centers.size(1),
              "data [m,k] and centers [n,k] must share k");
  TORCH_CHECK(x.scalar_type() == torch::kFloat32 && centers.scalar_type() == torch::kFloat32,
              "data and centers must be float32");
  c10::DeviceGuard guard(x.device());
  auto labels = torch::empty({x.size(0)}, torch::TensorOptions()
                                              .dtype(as_u8 ? torch::kUInt8 : torch::kInt64)
                                              .device(x.device()));
  check_rc(f2cgt_kmeans_predict(x.data_ptr<float>(), centers.data_ptr<float>(),
                                as_u8 ? nullptr : labels.data_ptr<int64_t>(),
                                as_u8 ? static_cast<uint8_t*>(labels.data_ptr()) : nullptr, x.size(0),
                                centers.size(0), x.size(1), metric_tag(metric), current_stream()),
           "kmeans_predict");
  return labels;
}

torch::Tensor pairwise_distance(torch::Tensor x, torch::Tensor y, std::string metric) {
  x = dev_contig(x, "x");
  y = dev_contig(y, "y");
  TORCH_CHECK(x.dim() == 2 && y.dim() == 2 && x.size(1) == y.size(1), "x [m,k] and y [n,k] must share k");
  TORCH_CHECK(x.scalar_type() == torch::kFloat32 && y.scalar_type() == torch::kFloat32,
              "x and y must be float32");
  c10::DeviceGuard guard(x.device());
  auto dist = empty_f32({x.size(0), y.size(0)}, x);
  check_rc(f2cgt_pairwise_distance(x.data_ptr<float>(), y.data_ptr<float>(), dist.data_ptr<float>(),
                                   x.size(0), y.size(0), x.size(1), metric_tag(metric), current_stream()),
           "pairwise_distance");
  return dist;
}

// Extension: one Lloyd centre update in place (the update half of examples/my_kmeans.py:87-113).
// -> shift fp32 [2] on the device = (sum_c |dc|, sum_c |dc|^2).  `stop` (int32 [1] on the device, optional)
// freezes the centres once `rule` is met (1: sum |dc|^2 < tol; 2: (sum |dc|)^2 < tol), see include/f2cgt.h.
torch::Tensor kmeans_update(torch::Tensor x, torch::Tensor labels, torch::Tensor centers,
                            c10::optional<torch::Tensor> stop, int64_t rule, double tol) {
  x = dev_contig(x, "data");
  labels = dev_contig(labels, "labels");
  TORCH_CHECK(centers.is_cuda() && centers.is_contiguous() && centers.scalar_type() == torch::kFloat32 &&
                  centers.dim() == 2,
              "centers must be a contiguous float32 GPU tensor [n, k] (it is updated in place)");
  TORCH_CHECK(x.dim() == 2 && x.scalar_type() == torch::kFloat32 && x.size(1) == centers.size(1),
              "data must be float32 [m, k]");
  TORCH_CHECK(labels.dim() == 1 && labels.size(0) == x.size(0) &&
                  (labels.scalar_type() == torch::kInt64 || labels.scalar_type() == torch::kUInt8),
              "labels must be int64 or uint8 [m]");
  int32_t* stop_ptr = nullptr;
  if (stop.has_value()) {
    TORCH_CHECK(stop->is_cuda() && stop->scalar_type() == torch::kInt32 && stop->numel() == 1,
                "stop must be an int32 GPU tensor with one element");
    stop_ptr = stop->data_ptr<int32_t>();
  }
  c10::DeviceGuard guard(x.device());
  const int64_t n = centers.size(0), k = centers.size(1);
  auto ws = torch::empty({f2cgt_kmeans_update_workspace_bytes(n, k)},
                         torch::TensorOptions().dtype(torch::kUInt8).device(x.device()));
  auto shift = empty_f32({2}, x);
  const bool u8 = labels.scalar_type() == torch::kUInt8;
  check_rc(f2cgt_kmeans_update(x.data_ptr<float>(), u8 ? nullptr : labels.data_ptr<int64_t>(),
                               u8 ? static_cast<const uint8_t*>(labels.data_ptr()) : nullptr,
                               centers.data_ptr<float>(), shift.data_ptr<float>(), stop_ptr, (int)rule, (float)tol,
                               ws.data_ptr(), ws.numel(), x.size(0), n, k, current_stream()),
           "kmeans_update");
  return shift;
}

// Counterpart of the reference's raft-backed KMeans (src/kmeans.h:13-31, src/kmeans.cu).
// predict() is the fused MFMA distance + arg-min kernel.  fit() is Lloyd's algorithm on the device:
// assignment (f2cgt_kmeans_predict) and centre update (f2cgt_kmeans_update) per iteration, stopped by
// raft's rule (sum of squared centre shifts below tol) which the update kernel evaluates itself; the
// host looks at the flag every eighth iteration only.  The centres start from distinct random rows
// (raft: random rows for cosine, k-means++ for L2; its RNG stream is not reproduced, so fit() is not a
// bit-parity target).  raft's batching and restart parameters have no counterpart here: a value other
// than the default draws a warning instead of being dropped silently.
class KMeans {
 public:
  KMeans(int64_t n_cluster, int64_t feat_dim, std::string metric, int max_iter, double tol, int n_init,
         double oversampling_factor, int batch_samples, int batch_centroids, bool inertia_check)
      : metric_(std::move(metric)), max_iter_(max_iter), tol_(tol), n_clusters_(n_cluster) {
    warn_ignored(n_init, oversampling_factor, batch_samples, batch_centroids, inertia_check);
    TORCH_CHECK(n_cluster > 0 && feat_dim > 0, "KMeans: n_cluster and feat_dim must be positive");
    centers_ = torch::zeros({n_cluster, feat_dim},
                            torch::TensorOptions().dtype(torch::kFloat32).device(torch::kCUDA));
  }
  KMeans(torch::Tensor centers, std::string metric, int max_iter, double tol, int n_init,
         double oversampling_factor, int batch_samples, int batch_centroids, bool inertia_check)
      : metric_(std::move(metric)), max_iter_(max_iter), tol_(tol) {
    warn_ignored(n_init, oversampling_factor, batch_samples, batch_centroids, inertia_check);
    TORCH_CHECK(centers.device().is_cuda(), "centers must be a CUDA tensor");
    TORCH_CHECK(centers.dim() == 2 && centers.scalar_type() == torch::kFloat32,
                "centers must be float32 [n_cluster, feat_dim]");
    centers_ = centers.contiguous();
    n_clusters_ = centers.size(0);
  }

  static void warn_ignored(int n_init, double oversampling_factor, int batch_samples, int batch_centroids,
                           bool inertia_check) {
    auto warn = [](const char* text) { py::module_::import("warnings").attr("warn")(std::string(text)); };
    if (n_init != 1) warn("KMeans: n_init is ignored (one run from one random start)");
    if (oversampling_factor != 2.0) warn("KMeans: oversampling_factor is ignored (no k-means|| seeding)");
    if (batch_samples != (1 << 15)) warn("KMeans: batch_samples is ignored (the kernels stream all rows)");
    if (batch_centroids != 0) warn("KMeans: batch_centroids is ignored (all centres are scored together)");
    if (inertia_check) warn("KMeans: inertia_check is ignored (the centre shift alone stops the fit)");
  }

  void fit(torch::Tensor x) {
    TORCH_CHECK(x.device().is_cuda(), "x must be a CUDA tensor");
    x = x.contiguous().to(torch::kFloat32);
    TORCH_CHECK(x.dim() == 2 && x.size(1) == centers_.size(1), "fit: data must be [n, feat_dim]");
    TORCH_CHECK(x.size(0) >= n_clusters_, "fit: fewer samples than clusters");
    c10::DeviceGuard guard(x.device());
    auto pick = torch::randperm(x.size(0), torch::TensorOptions().dtype(torch::kInt64).device(x.device()))
                    .slice(0, 0, n_clusters_);
    centers_.copy_(x.index_select(0, pick));
    auto stop = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt32).device(x.device()));
    const bool small = n_clusters_ <= 256;
    n_iter_ = 0;
    for (int it = 0; it < max_iter_; ++it) {
      auto labels = kmeans_predict_impl(x, centers_, metric_, small);
      kmeans_update(x, labels, centers_, stop, /*rule=*/1, tol_);
      ++n_iter_;
      if ((it & 7) == 7 && stop.item<int>() != 0) break;   // later steps are no-ops once the flag is up
    }
    // flag 2: the centre shift is not a number (NaN / infinite rows in the data); the centres are garbage
    TORCH_CHECK(stop.item<int>() != 2, "KMeans.fit: the centre shift became NaN (non-finite input rows?)");
  }

  int64_t n_iter() const { return n_iter_; }

  torch::Tensor predict(torch::Tensor x, bool normalize_weights) {
    (void)normalize_weights;  // sample weights only scale raft's inertia, never the labels
    TORCH_CHECK(x.device().is_cuda(), "x must be a CUDA tensor");
    return kmeans_predict_impl(x, centers_, metric_, false);
  }

  torch::Tensor get_centers() { return centers_; }

 private:
  std::string metric_;
  int max_iter_;
  double tol_;
  int64_t n_clusters_;
  int64_t n_iter_ = 0;
  torch::Tensor centers_;
};

// ---- extensions (not in the reference; defined by the benchmark configurations) -------

torch::Tensor affine_params_checked(torch::Tensor params, int64_t feat_dim) {
  params = dev_contig(params, "params");
  TORCH_CHECK(params.scalar_type() == torch::kFloat32 && params.dim() == 2 && params.size(0) == 2 &&
                  params.size(1) >= feat_dim,
              "affine params must be float32 [2, >= feat_dim] = (min, scale)");
  return params;
}

torch::Tensor sq_affine_decompress(torch::Tensor compress_data, torch::Tensor params, int64_t target_bits,
                                   int64_t feat_dim) {
  compress_data = dev_contig(compress_data, "compress_data");
  TORCH_CHECK(compress_data.dim() == 2 && (compress_data.scalar_type() == torch::kUInt8 ||
                                           compress_data.scalar_type() == torch::kInt8),
              "compress_data must be uint8 [rows, src_dim]");
  params = affine_params_checked(params, feat_dim);
  c10::DeviceGuard guard(compress_data.device());
  auto out = empty_f32({compress_data.size(0), feat_dim}, compress_data);
  check_rc(f2cgt_sq_affine_decompress(static_cast<const uint8_t*>(compress_data.data_ptr()),
                                      out.data_ptr<float>(), params.data_ptr<float>(), params.size(1),
                                      compress_data.size(0), compress_data.size(1), feat_dim,
                                      (int)target_bits, current_stream()),
           "sq_affine_decompress");
  return out;
}

torch::Tensor sq_affine_decompress_spmm_csr(torch::Tensor compress_feat, torch::Tensor params,
                                            torch::Tensor indptr, torch::Tensor indices,
                                            int64_t target_bit, int64_t feat_dim) {
  compress_feat = dev_contig(compress_feat, "compress_feat");
  TORCH_CHECK(compress_feat.dim() == 2 && (compress_feat.scalar_type() == torch::kUInt8 ||
                                           compress_feat.scalar_type() == torch::kInt8),
              "compress_feat must be uint8 [rows, src_dim]");
  params = affine_params_checked(params, feat_dim);
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(compress_feat.device());
  auto out = empty_f32({g.rows, feat_dim}, compress_feat);
  check_rc(f2cgt_sq_affine_decompress_spmm_csr(
               static_cast<const uint8_t*>(compress_feat.data_ptr()), params.data_ptr<float>(),
               params.size(1), g.indptr.data_ptr(), g.indices.data_ptr(), g.tag, out.data_ptr<float>(),
               g.rows, g.edges, compress_feat.size(0), compress_feat.size(1), feat_dim, (int)target_bit,
               current_stream()),
           "sq_affine_decompress_spmm_csr");
  return out;
}

torch::Tensor hybrid_decompress_spmm_csr(torch::Tensor row_map, torch::Tensor sq_codes,
                                         torch::Tensor sq_params, torch::Tensor vq_codes,
                                         torch::Tensor vq_codebooks, torch::Tensor indptr,
                                         torch::Tensor indices, int64_t feat_dim) {
  row_map = dev_contig(row_map, "row_map");
  sq_codes = dev_contig(sq_codes, "sq_codes");
  vq_codes = dev_contig(vq_codes, "vq_codes");
  vq_codebooks = dev_contig(vq_codebooks, "vq_codebooks");
  TORCH_CHECK(row_map.dim() == 1 && row_map.scalar_type() == torch::kInt32, "row_map must be int32 [n]");
  TORCH_CHECK(sq_codes.dim() == 2 && sq_codes.scalar_type() == torch::kUInt8 && sq_codes.size(1) == feat_dim,
              "sq_codes must be uint8 [n_sq, feat_dim]");
  TORCH_CHECK(vq_codes.dim() == 2 && vq_codes.scalar_type() == torch::kUInt8, "vq_codes must be uint8 [n_vq, n_codebooks]");
  TORCH_CHECK(vq_codebooks.dim() == 3 && vq_codebooks.scalar_type() == torch::kFloat32 &&
                  vq_codebooks.size(0) == vq_codes.size(1),
              "vq_codebooks must be float32 [n_codebooks, K, width]");
  sq_params = affine_params_checked(sq_params, feat_dim);
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(row_map.device());
  auto out = empty_f32({g.rows, feat_dim}, row_map);
  check_rc(f2cgt_hybrid_decompress_spmm_csr(
               row_map.data_ptr<int32_t>(), static_cast<const uint8_t*>(sq_codes.data_ptr()),
               sq_params.data_ptr<float>(), sq_params.size(1),
               static_cast<const uint8_t*>(vq_codes.data_ptr()), vq_codebooks.data_ptr<float>(),
               g.indptr.data_ptr(), g.indices.data_ptr(), g.tag, out.data_ptr<float>(), g.rows, g.edges,
               row_map.numel(), sq_codes.size(0), vq_codes.size(0), feat_dim, vq_codebooks.size(0),
               vq_codebooks.size(1), vq_codebooks.size(2), current_stream()),
           "hybrid_decompress_spmm_csr");
  return out;
}

void check_hip(hipError_t err, const char* what) {
  TORCH_CHECK(err == hipSuccess, what, ": ", hipGetErrorString(err));
}

// One extra stream (default priority) and its events per device, made on first use and kept for
// the life of the process.  Calls that overlap on one device from several host threads would share
// the events; the module is used from one thread per device like the reference's.
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t inputs_ready = nullptr, agg_done[2] = {nullptr, nullptr}, gemm_done[2] = {nullptr, nullptr};
};

SideStream* side_stream_of(int device) {
  static std::mutex lock;
  static std::map<int, SideStream> made;
  std::lock_guard<std::mutex> hold(lock);
  auto it = made.find(device);
  if (it != made.end()) return &it->second;
  SideStream s;
  check_hip(hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking), "hipStreamCreateWithFlags");
  for (hipEvent_t* ev : {&s.inputs_ready, &s.agg_done[0], &s.agg_done[1], &s.gemm_done[0], &s.gemm_done[1]})
    check_hip(hipEventCreateWithFlags(ev, hipEventDisableTiming), "hipEventCreateWithFlags");
  return &made.emplace(device, s).first->second;
}

// Aggregation followed by the dense layer that consumes it (the first layer of the GraphSAGE model,
// examples/conv.py:68-69, the layer examples/models.py:25-31 stacks, with the mean aggregator: h = fc_neigh(mean over the neighbours)).
// At the reference's widest shape (768 features -> 256 units, 341k destination rows) the fp32 GEMM
// takes 1.75 ms at 86 % of the matrix cores' fp32 peak and the aggregation 0.5 ms, so the multiply
// is not moved into the aggregation kernel: it would slow the part that already dominates.
//   block_rows == 0   one aggregation into a full-size buffer, one GEMM (the fastest form measured)
//   block_rows  > 0   destination rows in blocks of that many: the aggregate exists one block at a
//                     time, which bounds the extra memory to block_rows*feat_dim*4 bytes (1 GB at
//                     the shape above otherwise); ~6 % slower with 65536-row blocks
//   overlap           with blocks: the aggregation of block b+1 runs on a second stream beside the
//                     GEMM of block b, with two staging buffers.  Measured slower than running them
//                     one after the other (the two kernels contend for the same compute units), so
//                     it is off by default and kept for measurement.
// `agg(indptr_ptr, indices_ptr, rows, edges, dst, stream)` enqueues one block on `stream`.  With
// blocks the call reads the edge offsets of the block boundaries on the host, so it cannot be
// captured into a graph.
template <class Agg>
torch::Tensor aggregate_then_linear(const Graph& g, int64_t feat_dim, const torch::Tensor& like,
                                    torch::Tensor weight, const c10::optional<torch::Tensor>& bias,
                                    int64_t block_rows, bool overlap, Agg agg) {
  weight = dev_contig(weight, "weight");
  TORCH_CHECK(weight.dim() == 2 && weight.scalar_type() == torch::kFloat32 && weight.size(1) == feat_dim,
              "weight must be float32 [out_features, feat_dim]");
  torch::Tensor b;
  if (bias.has_value()) {
    b = dev_contig(*bias, "bias");
    TORCH_CHECK(b.dim() == 1 && b.scalar_type() == torch::kFloat32 && b.size(0) == weight.size(0),
                "bias must be float32 [out_features]");
  }
  TORCH_CHECK(block_rows >= 0, "block_rows must be >= 0 (0 = all rows at once)");
  auto out = empty_f32({g.rows, weight.size(0)}, like);
  if (g.rows == 0) return out;
  if (block_rows == 0) block_rows = g.rows;
  block_rows = std::min(block_rows, g.rows);
  const int64_t n_blocks = (g.rows + block_rows - 1) / block_rows;
  auto wt = weight.t();
  auto gemm = [&](torch::Tensor dst, const torch::Tensor& a) {
    if (b.defined())
      at::addmm_out(dst, b, a, wt);
    else
      at::mm_out(dst, a, wt);
  };
  if (n_blocks == 1) {
    auto whole = empty_f32({g.rows, feat_dim}, like);
    agg(g.indptr.data_ptr(), g.indices.data_ptr(), g.rows, g.edges, whole.data_ptr<float>(), current_stream());
    gemm(out, whole);
    return out;
  }
  // edge offsets at the block boundaries: the one host read of the call
  auto at_rows = torch::arange(0, n_blocks + 1, torch::TensorOptions().dtype(torch::kInt64).device(like.device()))
                     .mul_(block_rows).clamp_max_(g.rows);
  auto bounds = g.indptr.index_select(0, at_rows).to(torch::kInt64).cpu();
  const int64_t* e = bounds.data_ptr<int64_t>();
  TORCH_CHECK(e[0] >= 0 && e[n_blocks] <= g.edges, "indptr does not fit indices");
  for (int64_t blk = 0; blk < n_blocks; ++blk)
    TORCH_CHECK(e[blk] <= e[blk + 1], "indptr must be non-decreasing");

  // indptr of every block relative to the block's first edge (so that the kernel choice sees the
  // block's own degree), all blocks in one [n_blocks, block_rows + 1] tensor
  auto opts64 = torch::TensorOptions().dtype(torch::kInt64).device(like.device());
  auto pos = torch::arange(0, n_blocks, opts64).mul_(block_rows).unsqueeze(1) +
             torch::arange(0, block_rows + 1, opts64).unsqueeze(0);
  auto rebased = (g.indptr.index_select(0, pos.clamp_max_(g.rows).reshape({-1})).reshape({n_blocks, block_rows + 1}) -
                  bounds.slice(0, 0, n_blocks).to(like.device()).to(g.indptr.scalar_type()).unsqueeze(1))
                     .contiguous();

  const bool piped = overlap && n_blocks > 1;
  hipStream_t main_stream = static_cast<hipStream_t>(current_stream());
  SideStream* side = piped ? side_stream_of(like.device().index()) : nullptr;
  hipStream_t agg_stream = piped ? side->stream : main_stream;
  torch::Tensor stage[2];
  for (int i = 0; i < (piped ? 2 : 1); ++i) stage[i] = empty_f32({block_rows, feat_dim}, like);
  if (piped) {
    check_hip(hipEventRecord(side->inputs_ready, main_stream), "hipEventRecord");
    check_hip(hipStreamWaitEvent(agg_stream, side->inputs_ready, 0), "hipStreamWaitEvent");
  }
  const int64_t isz = g.indices.element_size(), psz = g.indptr.element_size();
  try {
  for (int64_t blk = 0; blk < n_blocks; ++blk) {
    const int64_t r0 = blk * block_rows, n = std::min(block_rows, g.rows - r0);
    const int slot = piped ? (int)(blk & 1) : 0;
    // the GEMM that last read this staging buffer must be over
    if (piped && blk >= 2) check_hip(hipStreamWaitEvent(agg_stream, side->gemm_done[slot], 0), "hipStreamWaitEvent");
    agg(static_cast<const char*>(rebased.data_ptr()) + blk * (block_rows + 1) * psz,
        static_cast<const char*>(g.indices.data_ptr()) + e[blk] * isz, n, e[blk + 1] - e[blk],
        stage[slot].data_ptr<float>(), static_cast<void*>(agg_stream));
    if (piped) {
      check_hip(hipEventRecord(side->agg_done[slot], agg_stream), "hipEventRecord");
      check_hip(hipStreamWaitEvent(main_stream, side->agg_done[slot], 0), "hipStreamWaitEvent");
    }
    gemm(out.narrow(0, r0, n), stage[slot].narrow(0, 0, n));
    if (piped) check_hip(hipEventRecord(side->gemm_done[slot], main_stream), "hipEventRecord");
  }
  } catch (...) {
    // a refused launch: nothing on the second stream may still use the staging buffers when they
    // are released
    if (piped) (void)hipStreamSynchronize(agg_stream);
    throw;
  }
  // every launch on the second stream is followed by a wait on the caller's stream, so the staging
  // buffers go back to the allocator under the caller's stream as usual
  return out;
}

torch::Tensor vq_decompress_spmm_csr_linear(torch::Tensor compress_feat, torch::Tensor codebooks,
                                            torch::Tensor indptr, torch::Tensor indices, int64_t feat_dim,
                                            torch::Tensor weight, c10::optional<torch::Tensor> bias,
                                            int64_t block_rows, bool overlap) {
  compress_feat = dev_contig(compress_feat, "compress_feat");
  codebooks = dev_contig(codebooks, "codebooks");
  TORCH_CHECK(compress_feat.dim() == 2, "compress_feat must be [rows, n_codebooks]");
  TORCH_CHECK(codebooks.dim() == 3 && codebooks.scalar_type() == torch::kFloat32,
              "VQ codebooks must be float32 [n_codebooks, K, width]");
  TORCH_CHECK(compress_feat.size(1) == codebooks.size(0), "compress_feat has ", compress_feat.size(1),
              " columns but there are ", codebooks.size(0), " codebooks");
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(compress_feat.device());
  const int tag = dtype_tag(compress_feat, "compress_feat");
  return aggregate_then_linear(
      g, feat_dim, compress_feat, weight, bias, block_rows, overlap,
      [&](const void* ip, const void* ix, int64_t rows, int64_t edges, float* dst, void* stream) {
        check_rc(f2cgt_vq_decompress_spmm_csr(compress_feat.data_ptr(), tag, codebooks.data_ptr<float>(), ip, ix,
                                              g.tag, dst, rows, edges, compress_feat.size(0), feat_dim,
                                              codebooks.size(0), codebooks.size(1), codebooks.size(2),
                                              stream),
                 "vq_decompress_spmm_csr_linear");
      });
}

torch::Tensor sq_decompress_spmm_csr_linear(torch::Tensor compress_feat, torch::Tensor codebooks,
                                            torch::Tensor indptr, torch::Tensor indices, int64_t target_bit,
                                            int64_t column_slice, int64_t feat_dim, torch::Tensor weight,
                                            c10::optional<torch::Tensor> bias, int64_t block_rows, bool overlap) {
  compress_feat = dev_contig(compress_feat, "compress_feat");
  TORCH_CHECK(compress_feat.dim() == 2, "compress_feat must be 2-D");
  codebooks = sq_codebooks_checked(codebooks);
  Graph g = graph_of(indptr, indices);
  c10::DeviceGuard guard(compress_feat.device());
  const int tag = dtype_tag(compress_feat, "compress_feat");
  return aggregate_then_linear(
      g, feat_dim, compress_feat, weight, bias, block_rows, overlap,
      [&](const void* ip, const void* ix, int64_t rows, int64_t edges, float* dst, void* stream) {
        check_rc(f2cgt_sq_decompress_spmm_csr(compress_feat.data_ptr(), tag, codebooks.data_ptr<float>(), ip, ix,
                                              g.tag, dst, rows, edges, compress_feat.size(0),
                                              compress_feat.size(1), feat_dim, codebooks.size(0), (int)target_bit,
                                              column_slice, stream),
                 "sq_decompress_spmm_csr_linear");
      });
}

torch::Tensor kmeans_predict(torch::Tensor x, torch::Tensor centers, std::string metric) {
  return kmeans_predict_impl(x, centers, metric, false);
}

// Row fetch of the feature cache (examples/tensor_cache.py:49-58).  `table` is a device tensor
// or a pinned host tensor (mapped into the device address space); `hot` and `slot_map` are the
// device-resident cache of hot rows and the id -> cache slot array (-1 = not cached).
torch::Tensor fetch_rows(torch::Tensor table, torch::Tensor index, c10::optional<torch::Tensor> hot,
                         c10::optional<torch::Tensor> slot_map) {
  TORCH_CHECK(table.defined() && table.dim() == 2 && table.is_contiguous(), "table must be a contiguous 2-D tensor");
  TORCH_CHECK(table.device().is_cuda() || table.is_pinned(),
              "table must be on the GPU or in pinned host memory");
  index = dev_contig(index, "index");
  TORCH_CHECK(index.dim() == 1, "index must be 1-D");
  auto st = index.scalar_type();
  TORCH_CHECK(st == torch::kInt64 || st == torch::kInt32, "index must be int32 or int64");
  TORCH_CHECK(hot.has_value() == slot_map.has_value(), "hot and slot_map come together");
  torch::Tensor hot_t, slot_t;
  int64_t num_hot = 0;
  if (hot.has_value()) {
    hot_t = dev_contig(*hot, "hot");
    slot_t = dev_contig(*slot_map, "slot_map");
    TORCH_CHECK(hot_t.dim() == 2 && hot_t.size(1) == table.size(1) && hot_t.scalar_type() == table.scalar_type(),
                "hot must have the row shape and dtype of table");
    TORCH_CHECK(slot_t.scalar_type() == torch::kInt32 && slot_t.dim() == 1 && slot_t.numel() == table.size(0),
                "slot_map must be int32 with one entry per row of table");
    num_hot = hot_t.size(0);
  }
  TORCH_CHECK(index.numel() == 0 || table.size(0) > 0, "rows requested from an empty table");
  c10::DeviceGuard guard(index.device());
  auto out = torch::empty({index.numel(), table.size(1)}, table.options().device(index.device()).pinned_memory(false));
  const int64_t row_bytes = table.size(1) * (int64_t)table.element_size();
  check_rc(f2cgt_fetch_rows(table.data_ptr(), num_hot ? hot_t.data_ptr() : nullptr,
                            num_hot ? slot_t.data_ptr<int32_t>() : nullptr, index.data_ptr(),
                            st == torch::kInt64 ? F2CGT_DT_I64 : F2CGT_DT_I32, out.data_ptr(), index.numel(),
                            row_bytes, table.size(0), num_hot, current_stream()),
           "fetch_rows");
  return out;
}

torch::Tensor vq_encode(torch::Tensor x, torch::Tensor centers, std::string metric) {
  return kmeans_predict_impl(x, centers, metric, true);
}

}  // namespace

// Output store policy of the SQ aggregation operators: "auto" (by output size), "stream"
// (non-temporal stores whatever the size) or "cached" (plain stores); returns the previous one.
std::string set_store_mode(const std::string& mode) {
  static const char* names[] = {"auto", "stream", "cached"};
  int want = -1;
  for (int i = 0; i < 3; ++i)
    if (mode == names[i]) want = i;
  TORCH_CHECK(want >= 0, "set_store_mode: mode must be \"auto\", \"stream\" or \"cached\", got \"", mode, "\"");
  const int was = f2cgt_set_store_mode(want);
  TORCH_CHECK(was >= 0, f2cgt_last_error());
  return names[was];
}

PYBIND11_MODULE(F2CGTLib, m) {
  m.doc() = "MI355X-native drop-in for F2CGT's F2CGTLib operator module";
  m.def("packbits", &packbits, py::arg("unpack"), py::arg("target_bits"))
      .def("unpackbits", &unpackbits, py::arg("pack"), py::arg("target_bits"), py::arg("unpack_dim"))
      .def("sq_compress", &sq_compress, py::arg("src"), py::arg("codebooks"), py::arg("target_bits"),
           py::arg("column_slice"))
      .def("sq_decompress", &sq_decompress, py::arg("compress_data"), py::arg("codebooks"),
           py::arg("target_bits"), py::arg("column_slice"), py::arg("feat_dim"))
      .def("vq_decompress", &vq_decompress, py::arg("index_tensor"), py::arg("codebooks"),
           py::arg("feat_dim"))
      .def("pairwise_distance", &pairwise_distance, py::arg("x"), py::arg("y"), py::arg("metric"))
      .def("spmm_csr", &spmm_csr, py::arg("feat"), py::arg("indptr"), py::arg("indices"))
      .def("vq_decompress_spmm_csr", &vq_decompress_spmm_csr, py::arg("compress_feat"),
           py::arg("codebooks"), py::arg("indptr"), py::arg("indices"), py::arg("feat_dim"))
      .def("sq_decompress_spmm_csr", &sq_decompress_spmm_csr, py::arg("compress_feat"),
           py::arg("codebooks"), py::arg("indptr"), py::arg("indices"), py::arg("target_bit"),
           py::arg("column_slice"), py::arg("feat_dim"));
  // extensions
  m.def("sq_affine_decompress", &sq_affine_decompress, py::arg("compress_data"), py::arg("params"),
        py::arg("target_bits"), py::arg("feat_dim"))
      .def("sq_affine_decompress_spmm_csr", &sq_affine_decompress_spmm_csr, py::arg("compress_feat"),
           py::arg("params"), py::arg("indptr"), py::arg("indices"), py::arg("target_bit"),
           py::arg("feat_dim"))
      .def("hybrid_decompress_spmm_csr", &hybrid_decompress_spmm_csr, py::arg("row_map"),
           py::arg("sq_codes"), py::arg("sq_params"), py::arg("vq_codes"), py::arg("vq_codebooks"),
           py::arg("indptr"), py::arg("indices"), py::arg("feat_dim"))
      .def("vq_decompress_spmm_csr_linear", &vq_decompress_spmm_csr_linear, py::arg("compress_feat"),
           py::arg("codebooks"), py::arg("indptr"), py::arg("indices"), py::arg("feat_dim"),
           py::arg("weight"), py::arg("bias") = py::none(), py::arg("block_rows") = 0, py::arg("overlap") = false)
      .def("sq_decompress_spmm_csr_linear", &sq_decompress_spmm_csr_linear, py::arg("compress_feat"),
           py::arg("codebooks"), py::arg("indptr"), py::arg("indices"), py::arg("target_bit"),
           py::arg("column_slice"), py::arg("feat_dim"), py::arg("weight"), py::arg("bias") = py::none(),
           py::arg("block_rows") = 0, py::arg("overlap") = false)
      .def("sq_encode", &sq_encode, py::arg("src"), py::arg("codebooks"), py::arg("target_bits"),
           py::arg("column_slice"))
      .def("kmeans_predict", &kmeans_predict, py::arg("x"), py::arg("centers"), py::arg("metric"))
      .def("vq_encode", &vq_encode, py::arg("x"), py::arg("centers"), py::arg("metric"))
      .def("fetch_rows", &fetch_rows, py::arg("table"), py::arg("index"), py::arg("hot") = py::none(),
           py::arg("slot_map") = py::none())
      .def("kmeans_update", &kmeans_update, py::arg("data"), py::arg("labels"), py::arg("centers"),
           py::arg("stop") = py::none(), py::arg("rule") = 0, py::arg("tol") = 0.0)
      .def("set_store_mode", &set_store_mode, py::arg("mode"));
  py::class_<KMeans>(m, "KMeans")
      .def(py::init<int64_t, int64_t, std::string, int, double, int, double, int, int, bool>(),
           py::arg("n_cluster"), py::arg("feat_dim"), py::arg("metric"), py::arg("max_iter") = 300,
           py::arg("tol") = 1e-4, py::arg("n_init") = 1, py::arg("oversampling_factor") = 2.0,
           py::arg("batch_samples") = 1 << 15, py::arg("batch_centroids") = 0,
           py::arg("inertia_check") = false)
      .def(py::init<torch::Tensor, std::string, int, double, int, double, int, int, bool>(),
           py::arg("centers"), py::arg("metric"), py::arg("max_iter") = 300, py::arg("tol") = 1e-4,
           py::arg("n_init") = 1, py::arg("oversampling_factor") = 2.0,
           py::arg("batch_samples") = 1 << 15, py::arg("batch_centroids") = 0,
           py::arg("inertia_check") = false)
      .def("fit", &KMeans::fit, py::arg("data"))
      .def("predict", &KMeans::predict, py::arg("data"), py::arg("normalize_weights") = true)
      .def("get_centers", &KMeans::get_centers)
      .def_property_readonly("n_iter", &KMeans::n_iter);   // extension: update steps issued by the last fit()
}
