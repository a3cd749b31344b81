// C[M,N] = A[M,K] * W[N,K]^T (+ bias) in bfloat16 with float accumulation through the vendor's library
// (hipBLASLt), called directly: the description of a product and its algorithm are made once per shape and
// kept, so that a call costs the host a few microseconds.  The algorithm is the heuristic's first choice at
// first.  A big product whose shape is worth it (the caller says so: the step is about to be recorded into a
// graph; or the shape has come up many times) gets the fastest of the heuristic's candidates instead, each
// run a few times on the operands of that call.  The reference's engine uses a library for its matrix
// products as well.  No device code here.
#include <hip/hip_runtime.h>
#include <hipblaslt/hipblaslt.h>

#include <cstdint>
#include <algorithm>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace {

struct Shape {
  int device, m, n, k, lda, ldc, bias;
  bool operator==(const Shape& o) const {
    return device == o.device && m == o.m && n == o.n && k == o.k && lda == o.lda && ldc == o.ldc && bias == o.bias;
  }
};
struct ShapeHash {
  size_t operator()(const Shape& s) const {
    uint64_t h = 1469598103934665603ull;
    for (int v : {s.device, s.m, s.n, s.k, s.lda, s.ldc, s.bias}) h = (h ^ (uint64_t)(uint32_t)v) * 1099511628211ull;
    return (size_t)h;
  }
};
struct Plan {
  hipblasLtMatmulDesc_t desc = nullptr;
  hipblasLtMatrixLayout_t w = nullptr, x = nullptr, c = nullptr;
  std::vector<hipblasLtMatmulHeuristicResult_t> candidates;   // those that fit the workspace, best guess first
  size_t chosen = 0;
  bool usable = false, tuned = false;
  int calls = 0;
};

std::mutex guard;
std::unordered_map<int, hipblasLtHandle_t> handles;       // one per device
std::unordered_map<Shape, Plan, ShapeHash> plans;
bool tuning = true;
// Multiply-adds from which the candidates are timed (a small product keeps the first choice: timed on operands
// that sit in the caches it would be misjudged).
constexpr double TUNE_FROM_WORK = 1073741824.0;
constexpr int TUNE_AFTER_CALLS = 64;                      // ... unasked, once a shape has come up this often

// The operands of the call that makes a plan: what the candidates are timed on.
struct Operands {
  const void* a; const void* w; const void* bias; void* c;
  void* workspace; size_t workspace_bytes; hipStream_t stream;
};

// Milliseconds of one product with this algorithm, the best of `runs`, each with cold caches: before every run
// `flush` (more bytes than the caches hold) is overwritten, which also keeps the device busy long enough for the
// host to have the product queued behind it, so that the two events bracket the product's own time on the device.
// In a model's step the weights of a product come from memory, not from the caches: candidates timed on operands
// that stay in the caches rank differently, and wrongly.  Negative if anything fails.
float time_algo(hipblasLtHandle_t handle, const Plan& p, const hipblasLtMatmulAlgo_t& algo, const Operands& o,
                void* flush, size_t flush_bytes, hipEvent_t start, hipEvent_t stop, int runs) {
  const float one = 1.f, zero = 0.f;
  float best = -1.f;
  for (int i = 0; i < runs; ++i) {
    float ms = -1.f;
    if (hipMemsetAsync(flush, i, flush_bytes, o.stream) != hipSuccess ||
        hipEventRecord(start, o.stream) != hipSuccess ||
        hipblasLtMatmul(handle, p.desc, &one, o.w, p.w, o.a, p.x, &zero, o.c, p.c, o.c, p.c, &algo, o.workspace,
                        o.workspace_bytes, o.stream) != HIPBLAS_STATUS_SUCCESS ||
        hipEventRecord(stop, o.stream) != hipSuccess || hipEventSynchronize(stop) != hipSuccess ||
        hipEventElapsedTime(&ms, start, stop) != hipSuccess)
      return -1.f;
    if (best < 0.f || ms < best) best = ms;
  }
  return best;
}

// Row-major C = A W^T is, in the library's column-major terms, C^T [N x M] = op(W) [N x K] * A^T [K x M]:
// W as stored is a K x N column-major matrix (transposed by the operation), A as stored a K x M one.
Plan make_plan(hipblasLtHandle_t handle, const Shape& s, size_t workspace_bytes) {
  Plan p;
  if (hipblasLtMatmulDescCreate(&p.desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) != HIPBLAS_STATUS_SUCCESS) return p;
  const hipblasOperation_t trans = HIPBLAS_OP_T, plain = HIPBLAS_OP_N;
  hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSA, &trans, sizeof(trans));
  hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_TRANSB, &plain, sizeof(plain));
  if (s.bias) {
    const hipblasLtEpilogue_t epilogue = HIPBLASLT_EPILOGUE_BIAS;
    const hipDataType bias_type = HIP_R_32F;
    const void* placeholder = nullptr;       // the pointer is set at every call
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_EPILOGUE, &epilogue, sizeof(epilogue));
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_DATA_TYPE, &bias_type, sizeof(bias_type));
    hipblasLtMatmulDescSetAttribute(p.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &placeholder, sizeof(placeholder));
  }
  if (hipblasLtMatrixLayoutCreate(&p.w, HIP_R_16BF, s.k, s.n, s.k) != HIPBLAS_STATUS_SUCCESS) return p;
  if (hipblasLtMatrixLayoutCreate(&p.x, HIP_R_16BF, s.k, s.m, s.lda) != HIPBLAS_STATUS_SUCCESS) return p;
  if (hipblasLtMatrixLayoutCreate(&p.c, HIP_R_16BF, s.n, s.m, s.ldc) != HIPBLAS_STATUS_SUCCESS) return p;
  hipblasLtMatmulPreference_t pref = nullptr;
  if (hipblasLtMatmulPreferenceCreate(&pref) != HIPBLAS_STATUS_SUCCESS) return p;
  hipblasLtMatmulPreferenceSetAttribute(pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &workspace_bytes,
                                        sizeof(workspace_bytes));
  // The heuristic's first choice may want more workspace than it was told there is: the first that fits is taken.
  constexpr int CANDIDATES = 24;
  hipblasLtMatmulHeuristicResult_t found[CANDIDATES];
  int count = 0;
  const hipblasStatus_t status =
      hipblasLtMatmulAlgoGetHeuristic(handle, p.desc, p.w, p.x, p.c, p.c, pref, CANDIDATES, found, &count);
  hipblasLtMatmulPreferenceDestroy(pref);
  if (status != HIPBLAS_STATUS_SUCCESS) return p;
  for (int i = 0; i < count; ++i)
    if (found[i].state == HIPBLAS_STATUS_SUCCESS && found[i].workspaceSize <= workspace_bytes)
      p.candidates.push_back(found[i]);
  p.usable = !p.candidates.empty();
  p.tuned = !tuning || p.candidates.size() < 2 || (double)s.m * s.n * s.k < TUNE_FROM_WORK;
  return p;
}

constexpr size_t FLUSH_BYTES = (size_t)384 << 20;        // more than the last-level caches hold together

// Time every candidate on these operands (the result they leave is the product all the same) and keep the
// fastest.  Not while the stream records a graph: the plan then stays as it is until a later call.
void tune_plan(hipblasLtHandle_t handle, Plan& p, const Operands& o) {
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(o.stream, &capture) != hipSuccess || capture != hipStreamCaptureStatusNone) return;
  p.tuned = true;
  void* flush = nullptr;
  hipEvent_t start = nullptr, stop = nullptr;
  if (hipMalloc(&flush, FLUSH_BYTES) == hipSuccess && hipEventCreate(&start) == hipSuccess &&
      hipEventCreate(&stop) == hipSuccess) {
    // Two rounds: every candidate three times, then the four fastest eight times more (candidates a few per cent
    // apart change places from one short measurement to the next, and the choice stays for the process's life).
    std::vector<std::pair<float, size_t>> ranked;
    for (size_t i = 0; i < p.candidates.size(); ++i) {
      const float ms = time_algo(handle, p, p.candidates[i].algo, o, flush, FLUSH_BYTES, start, stop, 3);
      if (ms >= 0.f) ranked.emplace_back(ms, i);
    }
    std::sort(ranked.begin(), ranked.end());
    float best_ms = -1.f;
    for (size_t r = 0; r < ranked.size() && r < 4; ++r) {
      const size_t i = ranked[r].second;
      float ms = time_algo(handle, p, p.candidates[i].algo, o, flush, FLUSH_BYTES, start, stop, 8);
      if (ms < 0.f) continue;
      ms = std::min(ms, ranked[r].first);
      if (best_ms < 0.f || ms < best_ms) { best_ms = ms; p.chosen = i; }
    }
    hipStreamSynchronize(o.stream);
  }
  if (start) hipEventDestroy(start);
  if (stop) hipEventDestroy(stop);
  if (flush) hipFree(flush);
  (void)hipGetLastError();                                  // a failed allocation leaves no error behind
}

}  // namespace

// A, W, C bfloat16 (rows of A `lda` apart, of C `ldc`), bias float32 [N] or null; `workspace`: device memory
// the library may use (the same for every call; products on one stream follow one another); `tune`: this
// shape will come again and again (its step is about to be recorded), so the choice of algorithm is worth timing.
// Returns 0; -3 if the library offers no algorithm for the shape (the caller uses a kernel of its own);
// -1 for arguments that make no sense; 1000 + the library's status for its errors.
extern "C" int ta_library_gemm_bf16(const void* A, const void* W, const void* bias, void* C, int M, int N, int K,
                                    int lda, int ldc, void* workspace, size_t workspace_bytes, int tune, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N || !A || !W || !C) return -1;
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return -1;
  std::lock_guard<std::mutex> lock(guard);
  auto handle_at = handles.find(device);
  if (handle_at == handles.end()) {
    hipblasLtHandle_t handle = nullptr;
    const hipblasStatus_t status = hipblasLtCreate(&handle);
    if (status != HIPBLAS_STATUS_SUCCESS) return 1000 + (int)status;
    handle_at = handles.emplace(device, handle).first;
  }
  const Shape shape{device, M, N, K, lda, ldc, bias ? 1 : 0};
  auto plan_at = plans.find(shape);
  if (plan_at == plans.end()) plan_at = plans.emplace(shape, make_plan(handle_at->second, shape, workspace_bytes)).first;
  Plan& plan = plan_at->second;
  if (!plan.usable) return -3;
  if (bias)
    hipblasLtMatmulDescSetAttribute(plan.desc, HIPBLASLT_MATMUL_DESC_BIAS_POINTER, &bias, sizeof(bias));
  if (!plan.tuned && (tune || ++plan.calls >= TUNE_AFTER_CALLS))
    tune_plan(handle_at->second, plan, Operands{A, W, bias, C, workspace, workspace_bytes, stream});
  const hipblasLtMatmulHeuristicResult_t& choice = plan.candidates[plan.chosen];
  const float one = 1.f, zero = 0.f;
  const hipblasStatus_t status =
      hipblasLtMatmul(handle_at->second, plan.desc, &one, W, plan.w, A, plan.x, &zero, C, plan.c, C, plan.c,
                      &choice.algo, workspace, workspace_bytes, stream);
  return status == HIPBLAS_STATUS_SUCCESS ? 0 : 1000 + (int)status;
}

// Whether plans made from now on time the heuristic's candidates (the default) or take its first choice.
extern "C" int ta_library_gemm_tuning(int on) {
  std::lock_guard<std::mutex> lock(guard);
  tuning = on != 0;
  return 0;
}
