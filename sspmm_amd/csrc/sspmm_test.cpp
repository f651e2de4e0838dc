// Benchmark / verification driver with the command line of the reference's sspmm_test
// (reference SSpMM/sspmm_test.cpp:289-350):
//
//   sspmm_test <paths.txt> <N> <V> <kernel> <sorted> <func> <mixed> <record> <reorder> <arch>
//
// Every line of paths.txt names a CVSE pattern file (what RowMerge writes) below
// $SSPMM_BENCHMARK_DIR (default "../benchmark") in dlmc-v<V>/ (reorder = 0) or dataset-v<V>/
// (reorder = 1).  As in the reference the values and the dense matrix are U(-1, 1) from a
// default-seeded engine, 200 launches are timed after 10 warm-ups, the figure is useful
// GFLOP/s = 2 * nnz * N / t, `func` checks against the host loop and `record` appends
// "nnz,m_vec,K,N,GFLOP/s" (plus bytes, GB/s and the fraction of the 8 TB/s HBM peak) to
// ./data/<arch>_rospmm_<V>_v<reorder>.csv.  kernel ids 0 and 1 run the same gfx950 kernels.
//
//   sspmm_test --synthetic <M> <K> <V> <sparsity> <N> [mixed] [func]
// runs one seeded vector-sparse matrix without any file.
//
// With `func` the process exits with status 2 when any matrix disagrees with the host loop: an element
// off by more than the reference's absolute 0.5 (reference SSpMM/sspmm_test.cpp:239), or a maximum
// error above $SSPMM_REL_TOL (default 1e-2) of the largest reference magnitude.
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <numeric>
#include <random>
#include <string>
#include <vector>

#include "../../include/sspmm.hpp"

namespace {

constexpr int kRepeat = 200, kWarmup = 10;
constexpr double kHbmPeakGBs = 8000.0;

void check(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    std::fprintf(stderr, "%s: %s\n", what, hipGetErrorString(e));
    std::exit(1);
  }
}

// U(-1, 1) from a copy of the caller's engine: consecutive calls see the same leading sequence,
// as with the by-value generator of the reference (SSpMM/include/bm_test_utils.h:140-152).
void make_dense(int64_t count, std::vector<__half> &out, std::default_random_engine generator) {
  std::uniform_real_distribution<float> dist(-1.0f, 1.0f);
  out.resize(count);
  for (int64_t i = 0; i < count; ++i) out[i] = __float2half(dist(generator));
}

struct Pattern {
  int m_vec = 0, K = 0;
  long long nnz = 0;  // scalar non-zeros of the original matrix: the "useful" count
  std::vector<int> row_offsets, col_indices;
};

bool read_cvse(const std::string &path, Pattern &p) {
  std::ifstream in(path);
  if (!in) return false;
  std::string line;
  std::getline(in, line, ',');
  p.m_vec = std::stoi(line);
  std::getline(in, line, ',');
  p.K = std::stoi(line);
  std::getline(in, line, '\n');
  p.nnz = std::stoll(line);
  p.row_offsets.resize(p.m_vec + 1);
  for (int i = 0; i <= p.m_vec; ++i) in >> p.row_offsets[i];
  p.col_indices.resize(p.row_offsets[p.m_vec]);
  for (auto &c : p.col_indices) in >> c;
  return !in.fail() || p.col_indices.empty();
}

Pattern synthetic_pattern(int M, int K, int V, double sparsity, unsigned seed) {
  Pattern p;
  p.m_vec = (M + V - 1) / V;
  p.K = K;
  const int per_row = std::max(0, std::min(K, (int)std::lround((1.0 - sparsity) * K)));
  std::mt19937_64 rng(seed);
  std::vector<int> perm(K);
  p.row_offsets.assign(1, 0);
  for (int i = 0; i < p.m_vec; ++i) {
    std::iota(perm.begin(), perm.end(), 0);
    for (int j = 0; j < per_row; ++j) std::swap(perm[j], perm[j + rng() % (K - j)]);
    std::sort(perm.begin(), perm.begin() + per_row);
    p.col_indices.insert(p.col_indices.end(), perm.begin(), perm.begin() + per_row);
    p.row_offsets.push_back((int)p.col_indices.size());
  }
  p.nnz = (long long)p.col_indices.size() * V;
  return p;
}

template <typename OutT>
float to_float(OutT v);
template <>
float to_float<float>(float v) { return v; }
template <>
float to_float<__half>(__half v) { return __half2float(v); }

// What this device sustains for a plain copy (reads + writes of 1 GiB each way), measured once per run: the
// denominator beside the published HBM peak.
double device_copy_gbs() {
  static double gbs = 0;
  if (gbs > 0) return gbs;
  const size_t bytes = (size_t)1 << 30;
  void *src = nullptr, *dst = nullptr;
  if (hipMalloc(&src, bytes) != hipSuccess || hipMalloc(&dst, bytes) != hipSuccess) {
    (void)hipFree(src);
    (void)hipGetLastError();
    return gbs = -1;
  }
  check(hipMemset(src, 1, bytes), "memset");
  hipEvent_t a, b;
  check(hipEventCreate(&a), "event");
  check(hipEventCreate(&b), "event");
  for (int i = 0; i < 3; ++i) check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, nullptr), "copy");
  check(hipEventRecord(a), "record");
  const int reps = 20;
  for (int i = 0; i < reps; ++i) check(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, nullptr), "copy");
  check(hipEventRecord(b), "record");
  check(hipEventSynchronize(b), "sync");
  float ms = 0;
  check(hipEventElapsedTime(&ms, a, b), "elapsed");
  check(hipEventDestroy(a), "event");
  check(hipEventDestroy(b), "event");
  (void)hipFree(src);
  (void)hipFree(dst);
  gbs = 2.0 * bytes * reps / ms / 1e6;
  std::printf("Device copy of 1 GiB: %.1f GB/s (reads + writes) = %.1f %% of the HBM peak\n", gbs, 100.0 * gbs / kHbmPeakGBs);
  return gbs;
}

double relative_tolerance() {
  const char *t = std::getenv("SSPMM_REL_TOL");
  const double v = t ? std::atof(t) : 0.0;
  return v > 0 ? v : 1e-2;
}

// Returns false when `func` is set and the result disagrees with the host loop.
template <typename OutT>
bool bench(const Pattern &p, int N, int V, int kernel, bool sorted, bool func, bool record, bool reorder,
           const std::string &arch) {
  const int m_vec = p.m_vec, K = p.K, M = m_vec * V;
  const int nvec = p.row_offsets[m_vec];
  std::default_random_engine generator;
  std::vector<__half> rhs, values;
  make_dense((int64_t)K * N, rhs, generator);
  make_dense((int64_t)nvec * V, values, generator);

  std::vector<float> host;
  if (func) {  // the reference's host loop (sspmm_test.cpp:75-95)
    host.assign((size_t)M * N, 0.0f);
    for (int i = 0; i < m_vec; ++i)
      for (int j = p.row_offsets[i]; j < p.row_offsets[i + 1]; ++j) {
        const int col = p.col_indices[j];
        for (int v = 0; v < V; ++v) {
          const float a = __half2float(values[(size_t)j * V + v]);
          float *c = &host[((size_t)i * V + v) * N];
          const __half *b = &rhs[(size_t)col * N];
          for (int l = 0; l < N; ++l) c[l] += a * __half2float(b[l]);
        }
      }
  }

  int *d_off, *d_col, *d_perm;
  __half *d_val, *d_rhs;
  OutT *d_out;
  check(hipMalloc(&d_off, (m_vec + 1) * sizeof(int)), "hipMalloc");
  check(hipMalloc(&d_col, std::max(nvec, 1) * sizeof(int)), "hipMalloc");
  check(hipMalloc(&d_perm, std::max(m_vec, 1) * sizeof(int)), "hipMalloc");
  check(hipMalloc(&d_val, std::max<size_t>((size_t)nvec * V, 1) * sizeof(__half)), "hipMalloc");
  check(hipMalloc(&d_rhs, std::max<size_t>((size_t)K * N, 1) * sizeof(__half)), "hipMalloc");
  check(hipMalloc(&d_out, std::max<size_t>((size_t)M * N, 1) * sizeof(OutT)), "hipMalloc");
  check(hipMemcpy(d_off, p.row_offsets.data(), (m_vec + 1) * sizeof(int), hipMemcpyHostToDevice), "copy");
  check(hipMemcpy(d_col, p.col_indices.data(), nvec * sizeof(int), hipMemcpyHostToDevice), "copy");
  check(hipMemcpy(d_val, values.data(), (size_t)nvec * V * sizeof(__half), hipMemcpyHostToDevice), "copy");
  check(hipMemcpy(d_rhs, rhs.data(), (size_t)K * N * sizeof(__half), hipMemcpyHostToDevice), "copy");
  if (sorted) {  // SortedRowSwizzle (bm_test_utils.h:210-225), on the device
    check((hipError_t)sspmm_sorted_row_swizzle(m_vec, d_off, d_perm, nullptr), "row swizzle");
  } else {
    std::vector<int> ident(m_vec);
    std::iota(ident.begin(), ident.end(), 0);
    check(hipMemcpy(d_perm, ident.data(), m_vec * sizeof(int), hipMemcpyHostToDevice), "copy");
  }

  std::printf(kernel == 0 ? "Using the SpMM entry point\n" : "Using the SSpMM entry point\n");
  hipEvent_t start, end;
  check(hipEventCreate(&start), "event");
  check(hipEventCreate(&end), "event");
  float total_msec = 0;
  for (int i = 0; i < kRepeat + kWarmup; ++i) {
    check(hipEventRecord(start), "record");
    const hipError_t rc = kernel == 0
                              ? spmm::SpMM(m_vec, V, N, K, d_perm, d_off, d_col, d_val, d_rhs, d_out)
                              : spmm::SSpMM(m_vec, V, N, K, d_perm, d_off, d_col, d_val, d_rhs, d_out);
    check(rc, "SSpMM");
    check(hipEventRecord(end), "record");
    check(hipEventSynchronize(end), "sync");
    float msec = 0;
    check(hipEventElapsedTime(&msec, start, end), "elapsed");
    if (i >= kWarmup) total_msec += msec;
  }
  check(hipEventDestroy(start), "event");
  check(hipEventDestroy(end), "event");

  const double ms = total_msec / kRepeat;
  const double gflops = (double)p.nnz * N * 2 / 1e6 / ms;
  const double bytes = 2.0 * V * nvec + 4.0 * nvec + 4.0 * (m_vec + 1) + 2.0 * K * N + sizeof(OutT) * (double)M * N;
  const double gbs = bytes / ms / 1e6;
  const double sp = M > 0 && K > 0 ? 100.0 - (double)p.nnz * 100 / M / K : 100.0;
  const double copy_gbs = device_copy_gbs();  // (prints its own line the first time)
  std::printf("M = %d, K = %d, N = %d, NNZ = %lld, Sparsity = %lf%%\n", M, K, N, p.nnz, sp);
  std::printf("Average Performance = %lf GFlops, %.3f us per launch, %.1f GB/s = %.1f %% of the HBM peak", gflops,
              ms * 1e3, gbs, 100.0 * gbs / kHbmPeakGBs);
  if (copy_gbs > 0) std::printf(", %.1f %% of the device's copy rate", 100.0 * gbs / copy_gbs);
  std::printf("\n");
  if (record) {
    const std::string path = "./data/" + arch + "_rospmm_" + std::to_string(V) + (reorder ? "_v1.csv" : "_v0.csv");
    std::ofstream out(path, std::ios::app);
    if (!out) std::fprintf(stderr, "cannot open %s (create ./data first)\n", path.c_str());
    out << p.nnz << ',' << m_vec << ',' << K << ',' << N << ',' << gflops << ',' << (long long)bytes << ',' << gbs
        << ',' << gbs / kHbmPeakGBs << std::endl;
  }
  bool agrees = true;
  if (func) {
    std::vector<OutT> got((size_t)M * N);
    check(hipMemcpy(got.data(), d_out, got.size() * sizeof(OutT), hipMemcpyDeviceToHost), "copy");
    int errors = 0;
    float max_error = 0, max_ref = 0;
    for (size_t j = 0; j < got.size(); ++j) {
      const float d = std::fabs(to_float(got[j]) - host[j]);
      max_error = std::max(max_error, d);
      max_ref = std::max(max_ref, std::fabs(host[j]));
      if (d > 0.5f) ++errors;  // the reference's threshold (sspmm_test.cpp:239)
    }
    const double rel = max_ref > 0 ? max_error / max_ref : max_error;
    if (errors || rel > relative_tolerance()) {
      std::printf("SPMM does not agree with SEQUENTIAL! %d errors! max error: %f (%g of max |ref|, tolerance %g)\n", errors,
                  max_error, rel, relative_tolerance());
      agrees = false;
    } else {
      std::printf("Results verified: they agree. max abs error %g, relative to max |ref| %g\n", max_error, rel);
    }
  }
  (void)hipFree(d_off);
  (void)hipFree(d_col);
  (void)hipFree(d_perm);
  (void)hipFree(d_val);
  (void)hipFree(d_rhs);
  (void)hipFree(d_out);
  return agrees;
}

void usage() {
  std::printf("sspmm_test <paths.txt> <dimN> <vec_length 8|16> <kernel 0|1> <sort 0|1> <verify 0|1> "
              "<mixed 0: fp32 out, 1: fp16 out> <record 0|1> <reorder 0|1> <arch>\n"
              "sspmm_test --synthetic <M> <K> <V> <sparsity> <N> [mixed] [verify]\n");
  std::exit(1);
}

}  // namespace

int main(int argc, char **argv) {
  if (argc >= 7 && std::strcmp(argv[1], "--synthetic") == 0) {
    const int M = std::atoi(argv[2]), K = std::atoi(argv[3]), V = std::atoi(argv[4]);
    const double sparsity = std::atof(argv[5]);
    const int N = std::atoi(argv[6]);
    const int mixed = argc > 7 ? std::atoi(argv[7]) : 0, func = argc > 8 ? std::atoi(argv[8]) : 1;
    const Pattern p = synthetic_pattern(M, K, V, sparsity, 1);
    const bool ok = mixed ? bench<__half>(p, N, V, 1, false, func, false, false, "gfx950")
                          : bench<float>(p, N, V, 1, false, func, false, false, "gfx950");
    return ok ? 0 : 2;
  }
  if (argc != 11) usage();
  const std::string paths(argv[1]);
  const int dimN = std::atoi(argv[2]), V = std::atoi(argv[3]), kernel = std::atoi(argv[4]);
  const int sorted = std::atoi(argv[5]), func = std::atoi(argv[6]), mixed = std::atoi(argv[7]);
  const int record = std::atoi(argv[8]), reorder = std::atoi(argv[9]);
  const std::string arch(argv[10]);
  if (kernel != 0 && kernel != 1) {
    std::printf("Unsupported Kernel \n");
    return 1;
  }
  const char *root = std::getenv("SSPMM_BENCHMARK_DIR");
  std::string dir = std::string(root ? root : "../benchmark") + "/";
  if (V == 8 || V == 16) dir += std::string(reorder ? "dataset-v" : "dlmc-v") + std::to_string(V) + "/";
  else dir += "dlmc/";
  std::ifstream list(paths);
  if (!list) {
    std::fprintf(stderr, "cannot open %s\n", paths.c_str());
    return 1;
  }
  std::string line;
  int count = 0, failed = 0;
  while (std::getline(list, line)) {
    if (line.empty()) continue;
    std::cout << "NO." << count << "  matrix:" << std::endl;
    Pattern p;
    if (!read_cvse(dir + line, p)) {
      std::fprintf(stderr, "cannot read %s\n", (dir + line).c_str());
      return 1;
    }
    const bool ok = mixed ? bench<__half>(p, dimN, V, kernel, sorted, func, record, reorder, arch)
                          : bench<float>(p, dimN, V, kernel, sorted, func, record, reorder, arch);
    if (!ok) ++failed;
    ++count;
  }
  std::printf("matrix num:%d\n", count);
  if (failed) {
    std::printf("%d of them disagree with the host loop\n", failed);
    return 2;
  }
  return 0;
}
