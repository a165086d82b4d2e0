// Python module `neoGEMM`: the PyTorch-ROCm face of libneogemm.so.
//
// Keeps the reference's extension surface — module neoGEMM, function neoGemmV1(A, B, C) with keyword
// names A, B, C returning None (nemgemmV03.cu:343-399, neogemmv4.cu:335-338), the older
// neogemm(A, B, C) (v01.cu:272-317, neogemmV02.cu:304-307) — and adds C = gemm(A, B).  This file
// only unwraps tensors, checks them and calls the C ABI of include/neogemm.h on torch's current HIP
// stream; there is no kernel code and no HIP call here apart from asking torch for that stream.
//
// Differences from the reference launcher, on purpose:
//  * arguments are validated (the reference only checks dtype through data_ptr<>, nemgemmV03.cu:349-351)
//    and failures raise instead of printing to stderr (nemgemmV03.cu:387-390);
//  * the launch goes to torch's current stream, not the legacy default stream (nemgemmV03.cu:383);
//  * no state tied to a tensor is cached between calls (the reference caches TMA descriptors keyed on shape
//    only, nemgemmV03.cu:27-30,359-371, which goes stale when another tensor of the same shape is passed); the
//    only state kept is a split-K scratch buffer per (device, stream).
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <map>
#include <string>

#include "neogemm.h"

namespace {

void check_operand(const torch::Tensor& t, const char* name) {
  TORCH_CHECK(t.defined(), name, " is undefined");
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(t.scalar_type() == at::kBFloat16, name, " must be bfloat16, got ", t.scalar_type());
  TORCH_CHECK(t.dim() == 2, name, " must be 2-D, got ", t.dim(), "-D");
}

// A 2-D tensor whose rows are contiguous (stride(1) == 1) is passed with ld = stride(0).
bool row_major(const torch::Tensor& t) { return t.size(1) <= 1 || t.stride(1) == 1; }
int64_t row_ld(const torch::Tensor& t) { return t.size(0) <= 1 ? std::max<int64_t>(t.size(1), 1) : t.stride(0); }

// Split-K scratch, one buffer per (device, stream): two GEMMs on two streams of one device must not share their
// partials, and a buffer is only ever used on the stream that was current when the caching allocator handed it out,
// which is the stream whose order the allocator follows when the block is reused.  So dropping a buffer that has
// become too small is safe: its block goes back to that stream's pool and is handed out again only to work queued
// on that same stream, behind the kernels that still use it.  The cache is per host thread.
struct WorkspaceKey {
  int device;
  hipStream_t stream;
  bool operator<(const WorkspaceKey& o) const { return device != o.device ? device < o.device : stream < o.stream; }
};
// At most kMaxWorkspaces buffers are kept: streams come and go, and a buffer whose stream is gone would otherwise stay
// for the life of the thread.  The least recently used one is dropped (safe for the reason above).
constexpr size_t kMaxWorkspaces = 16;
struct WorkspaceSlot {
  torch::Tensor buffer;
  uint64_t last_use = 0;
};
torch::Tensor& workspace_for(const torch::Tensor& like, hipStream_t stream, size_t bytes) {
  static thread_local std::map<WorkspaceKey, WorkspaceSlot> ws;
  static thread_local uint64_t clock = 0;
  const WorkspaceKey key{(int)like.get_device(), stream};
  if (ws.find(key) == ws.end() && ws.size() >= kMaxWorkspaces) {
    auto oldest = ws.begin();
    for (auto it = ws.begin(); it != ws.end(); ++it)
      if (it->second.last_use < oldest->second.last_use) oldest = it;
    ws.erase(oldest);
  }
  WorkspaceSlot& slot = ws[key];
  slot.last_use = ++clock;
  torch::Tensor& t = slot.buffer;
  if (!t.defined() || (size_t)t.numel() < bytes) {
    t = torch::Tensor();  // give the old block back first
    t = torch::empty({(int64_t)bytes}, like.options().dtype(torch::kUInt8));
  }
  return t;
}

void run(const torch::Tensor& A, const torch::Tensor& B, torch::Tensor& C, int64_t M, int64_t N, int64_t K,
         int64_t lda, int64_t ldb, int64_t ldc, int b_layout, int c_layout, float alpha = 1.f, float beta = 0.f) {
  // PyTorch-ROCm names its HIP devices "cuda"; these are the guard and stream accessors for that naming
  c10::hip::HIPGuardMasqueradingAsCUDA guard(A.device());
  const size_t need = neogemm_bf16_workspace_bytes(M, N, K);
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(A.get_device()).stream();
  void* ws = nullptr;
  if (need) ws = workspace_for(A, stream, need).data_ptr();
  const int st = (alpha == 1.f && beta == 0.f)
                     ? neogemm_bf16(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, ldc, b_layout,
                                    c_layout, ws, need, (void*)stream)
                     : neogemm_bf16_scaled(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, lda, ldb, ldc, b_layout,
                                           c_layout, alpha, beta, ws, need, (void*)stream);
  TORCH_CHECK(st == NEOGEMM_OK, "neogemm_bf16 failed: ", neogemm_strerror(st));
}

// C = gemm(A, B): A [M,K], B [K,N] -> new C [M,N], all bf16.  A transposed view of a contiguous
// [N,K] tensor is taken as is (that is the reference's own B layout), anything else is made contiguous.
torch::Tensor gemm(torch::Tensor A, torch::Tensor B) {
  check_operand(A, "A");
  check_operand(B, "B");
  TORCH_CHECK(A.device() == B.device(), "A and B must be on the same device");
  TORCH_CHECK(A.size(1) == B.size(0), "inner dimensions differ: A is ", A.sizes(), ", B is ", B.sizes());
  if (!row_major(A)) A = A.contiguous();
  int b_layout = NEOGEMM_B_KN;
  int64_t ldb;
  if (row_major(B)) {
    ldb = row_ld(B);
  } else if (B.stride(0) == 1) {  // B = W.t() with W [N,K] row-major
    b_layout = NEOGEMM_B_NK;
    ldb = B.size(1) <= 1 ? std::max<int64_t>(B.size(0), 1) : B.stride(1);
  } else {
    B = B.contiguous();
    ldb = row_ld(B);
  }
  const int64_t M = A.size(0), K = A.size(1), N = B.size(1);
  torch::Tensor C = torch::empty({M, N}, A.options());
  if (M == 0 || N == 0) return C;
  run(A, B, C, M, N, K, row_ld(A), ldb, std::max<int64_t>(N, 1), b_layout, NEOGEMM_C_ROW);
  return C;
}

// gemm_scaled(A, B, C, alpha, beta): C[M,N] (row-major, contiguous) = alpha * A[M,K] @ B[K,N] + beta * C, in place;
// the epilogue the reference's v4 kernel declares (neogemmv4.cu:166,266).
void gemm_scaled(torch::Tensor A, torch::Tensor B, torch::Tensor C, double alpha, double beta) {
  check_operand(A, "A");
  check_operand(B, "B");
  check_operand(C, "C");
  TORCH_CHECK(A.device() == B.device() && A.device() == C.device(), "A, B and C must be on the same device");
  TORCH_CHECK(A.size(1) == B.size(0), "inner dimensions differ: A is ", A.sizes(), ", B is ", B.sizes());
  TORCH_CHECK(C.size(0) == A.size(0) && C.size(1) == B.size(1) && C.is_contiguous(), "C must be a contiguous [M,N]");
  if (!row_major(A)) A = A.contiguous();
  int b_layout = NEOGEMM_B_KN;
  int64_t ldb;
  if (row_major(B)) {
    ldb = row_ld(B);
  } else if (B.stride(0) == 1) {
    b_layout = NEOGEMM_B_NK;
    ldb = B.size(1) <= 1 ? std::max<int64_t>(B.size(0), 1) : B.stride(1);
  } else {
    B = B.contiguous();
    ldb = row_ld(B);
  }
  const int64_t M = A.size(0), K = A.size(1), N = B.size(1);
  if (M == 0 || N == 0) return;
  run(A, B, C, M, N, K, row_ld(A), ldb, std::max<int64_t>(N, 1), b_layout, NEOGEMM_C_ROW, (float)alpha, (float)beta);
}

// bmm(A, B): A [b,M,K], B [b,K,N] or [K,N] (shared) -> new C [b,M,N]; one launch (neogemm_bf16_batched).
torch::Tensor bmm(torch::Tensor A, torch::Tensor B) {
  TORCH_CHECK(A.is_cuda() && B.is_cuda(), "A and B must be GPU tensors (there is no CPU path)");
  TORCH_CHECK(A.scalar_type() == torch::kBFloat16 && B.scalar_type() == torch::kBFloat16, "A and B must be bfloat16");
  TORCH_CHECK(A.dim() == 3 && (B.dim() == 3 || B.dim() == 2), "A must be [b,M,K], B [b,K,N] or [K,N]");
  TORCH_CHECK(A.device() == B.device(), "A and B must be on the same device");
  TORCH_CHECK(A.size(2) == B.size(B.dim() - 2) && (B.dim() == 2 || B.size(0) == A.size(0)), "shapes do not match: A ",
              A.sizes(), ", B ", B.sizes());
  A = A.contiguous();
  B = B.contiguous();
  const int64_t batch = A.size(0), M = A.size(1), K = A.size(2), N = B.size(B.dim() - 1);
  torch::Tensor C = torch::empty({batch, M, N}, A.options());
  if (batch == 0 || M == 0 || N == 0) return C;
  c10::hip::HIPGuardMasqueradingAsCUDA guard(A.device());
  const size_t need = neogemm_bf16_batched_workspace_bytes(M, N, K, batch);
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(A.get_device()).stream();
  void* ws = nullptr;
  if (need) ws = workspace_for(A, stream, need).data_ptr();
  const int st = neogemm_bf16_batched(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, std::max<int64_t>(K, 1),
                                      std::max<int64_t>(N, 1), std::max<int64_t>(N, 1), M * K, B.dim() == 3 ? K * N : 0,
                                      M * N, batch, NEOGEMM_B_KN, NEOGEMM_C_ROW, ws, need, (void*)stream);
  TORCH_CHECK(st == NEOGEMM_OK, "neogemm_bf16_batched failed: ", neogemm_strerror(st));
  return C;
}

// neoGemmV1(A, B, C): A [M,K], B [N,K], C holds M*N bf16 and receives the product column-major,
// so that C.t() (viewing the [M,N]-shaped C of benchmark.py:12 transposed, benchmark.py:25) equals
// A @ B.t() (benchmark.py:18) when M == N, and C.view(N, M).t() does in general.
void neoGemmV1(torch::Tensor A, torch::Tensor B, torch::Tensor C) {
  check_operand(A, "A");
  check_operand(B, "B");
  check_operand(C, "C");
  TORCH_CHECK(A.device() == B.device() && A.device() == C.device(), "A, B and C must be on the same device");
  TORCH_CHECK(A.size(1) == B.size(1), "A is [M,K] and B is [N,K]: K differs (", A.size(1), " vs ", B.size(1), ")");
  TORCH_CHECK(A.is_contiguous() && B.is_contiguous() && C.is_contiguous(), "A, B and C must be contiguous");
  const int64_t M = A.size(0), K = A.size(1), N = B.size(0);
  TORCH_CHECK(C.numel() == M * N, "C must hold M*N = ", M * N, " elements, has ", C.numel());
  if (M == 0 || N == 0) return;
  run(A, B, C, M, N, K, std::max<int64_t>(K, 1), std::max<int64_t>(K, 1), M, NEOGEMM_B_NK, NEOGEMM_C_COL);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "BF16 GEMM for MI355X (gfx950): bf16 in, fp32 accumulate, bf16 out";
  m.def("gemm", &gemm, "C[M,N] = A[M,K] @ B[K,N]", py::arg("A"), py::arg("B"));
  m.def("neoGemmV1", &neoGemmV1, "C (column-major) = A[M,K] @ B[N,K]^T, in place", py::arg("A"), py::arg("B"),
        py::arg("C"));
  m.def("neogemm", &neoGemmV1, "alias of neoGemmV1 (the reference's first module name)", py::arg("A"),
        py::arg("B"), py::arg("C"));
  m.def("gemm_scaled", &gemm_scaled, "C = alpha * A[M,K] @ B[K,N] + beta * C, in place", py::arg("A"), py::arg("B"),
        py::arg("C"), py::arg("alpha") = 1.0, py::arg("beta") = 0.0);
  m.def("bmm", &bmm, "C[b,M,N] = A[b,M,K] @ B[b,K,N] (or B [K,N] shared)", py::arg("A"), py::arg("B"));
  m.def("version", []() { return std::string(neogemm_version()); });
}
