// PyTorch-ROCm binding: module `grouped_gemm_backend`, one function
// gmm(a, b, c, batch_sizes, trans_a, trans_b) -> None, the same entry point the
// reference's extension exports (csrc/ops.cu:7-9, csrc/grouped_gemm.h:5-9).
//
// All tensor validation lives here, in the order of the reference's checks
// (csrc/grouped_gemm.cu:470-540, :437-460, :120-124), and runs before anything touches
// the device; the compute is one call into the C ABI of libgrouped_gemm_hip.so on
// torch's current HIP stream.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <torch/extension.h>

#include <map>
#include <mutex>
#include <utility>

#include "../../include/grouped_gemm_hip.h"

namespace grouped_gemm {

namespace {

bool IsFloat8(torch::ScalarType t) { return t == torch::kFloat8_e4m3fn || t == torch::kFloat8_e5m2; }

// Element type of c for operands of type `t`: the same for the two-byte types, bf16 for fp8.
torch::ScalarType OutputType(torch::ScalarType t) { return IsFloat8(t) ? torch::kBFloat16 : t; }

int DtypeCode(torch::ScalarType t) {
  switch (t) {
    case torch::kFloat16: return GG_DTYPE_F16;
    case torch::kFloat8_e4m3fn: return GG_DTYPE_F8E4M3;
    case torch::kFloat8_e5m2: return GG_DTYPE_F8E5M2;
    default: return GG_DTYPE_BF16;
  }
}

// Row indices of the fused gather / scatter forms (see gg_gmm): undefined tensors mean "rows in place".
struct RowIndices {
  torch::Tensor a, b, c;
  bool any() const { return a.defined() || b.defined() || c.defined(); }
};

// `on_device` false skips the checks that a tensor lives on the GPU, so that the shape,
// rank and dtype rules can be exercised with CPU tensors on a machine without one.
// With row indices, `tokens` (the rows of the product) is the length of the index instead of the
// row count of the tensor it redirects.
// With `gate_up`, b holds two matrices per expert side by side and c is half as wide as b.
void Validate(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& c,
              const torch::Tensor& batch_sizes, bool trans_a, bool trans_b, bool on_device,
              const RowIndices& rows = RowIndices(), bool gate_up = false) {
  // Only one of the operands may be transposed (csrc/grouped_gemm.cu:476).
  TORCH_CHECK(!(trans_a && trans_b), "grouped_gemm: trans_a and trans_b cannot both be set");

  // batch_sizes may live on the host or on the device (csrc/grouped_gemm.cu:478-486).
  TORCH_CHECK(batch_sizes.is_cuda() || batch_sizes.is_cpu(),
              "grouped_gemm: batch_sizes must be a CPU or GPU tensor");
  TORCH_CHECK(batch_sizes.ndimension() == 1, "grouped_gemm: batch_sizes must be 1-d");
  TORCH_CHECK(batch_sizes.scalar_type() == torch::kInt64, "grouped_gemm: batch_sizes must be int64");

  // a: (tokens, hidden_in) bf16 on the GPU (csrc/grouped_gemm.cu:490-492).  float16 is accepted
  // as well, for all three tensors alike; the reference takes bfloat16 only.
  if (on_device) TORCH_CHECK(a.is_cuda(), "grouped_gemm: a must be a GPU tensor");
  TORCH_CHECK(a.ndimension() == 2, "grouped_gemm: a must be 2-d");
  TORCH_CHECK(a.scalar_type() == torch::kBFloat16 || a.scalar_type() == torch::kFloat16 || IsFloat8(a.scalar_type()),
              "grouped_gemm: a must be bfloat16 (or float16, float8_e4m3fn, float8_e5m2)");

  // b, c: bf16 on the GPU (csrc/grouped_gemm.cu:503-506).
  if (on_device) {
    TORCH_CHECK(b.is_cuda(), "grouped_gemm: b must be a GPU tensor");
    TORCH_CHECK(c.is_cuda(), "grouped_gemm: c must be a GPU tensor");
  }
  TORCH_CHECK(b.scalar_type() == a.scalar_type(), "grouped_gemm: b must be bfloat16 (the element type of a)");
  TORCH_CHECK(c.scalar_type() == OutputType(a.scalar_type()),
              "grouped_gemm: c must be bfloat16 (the element type of a; bfloat16 for float8 operands)");
  for (const torch::Tensor* idx : {&rows.a, &rows.b, &rows.c}) {
    if (!idx->defined()) continue;
    TORCH_CHECK(idx->ndimension() == 1 && idx->scalar_type() == torch::kInt32 && idx->is_contiguous(),
                "grouped_gemm: a row index must be a contiguous 1-d int32 tensor");
    if (on_device) TORCH_CHECK(idx->is_cuda() && idx->device() == a.device(), "grouped_gemm: a row index must be on a's GPU");
  }
  TORCH_CHECK(!(trans_a && rows.c.defined()), "grouped_gemm: the trans_a output has no row per token to scatter");
  TORCH_CHECK(!(trans_a && gate_up), "grouped_gemm: the SwiGLU epilogue is not for the trans_a layout");
  TORCH_CHECK(trans_a || !rows.b.defined(), "grouped_gemm: only the trans_a layout has a row per token in b");
  const int64_t tokens = rows.a.defined() ? rows.a.size(0) : a.size(0);

  if (trans_a) {
    // b (tokens, hidden_out), c (num_experts, hidden_in, hidden_out)
    // (csrc/grouped_gemm.cu:513-522).
    TORCH_CHECK(b.ndimension() == 2, "grouped_gemm: with trans_a, b must be 2-d");
    TORCH_CHECK(c.ndimension() == 3, "grouped_gemm: with trans_a, c must be 3-d");
    TORCH_CHECK((rows.b.defined() ? rows.b.size(0) : b.size(0)) == tokens,
                "grouped_gemm: a and b must have the same number of rows");
    TORCH_CHECK(c.size(0) == batch_sizes.size(0), "grouped_gemm: c.size(0) must equal the number of experts");
    TORCH_CHECK(c.size(1) == a.size(1), "grouped_gemm: c.size(1) must equal a.size(1)");
    TORCH_CHECK(c.size(2) == b.size(1), "grouped_gemm: c.size(2) must equal b.size(1)");
  } else {
    // b (num_experts, hidden_in, hidden_out) or transposed, c (tokens, hidden_out)
    // (csrc/grouped_gemm.cu:524-534).
    TORCH_CHECK(b.ndimension() == 3, "grouped_gemm: b must be 3-d");
    TORCH_CHECK(c.ndimension() == 2, "grouped_gemm: c must be 2-d");
    const int64_t hidden_in = trans_b ? b.size(2) : b.size(1);
    TORCH_CHECK(hidden_in == a.size(1), "grouped_gemm: contraction dimensions of a and b differ");
    TORCH_CHECK(batch_sizes.size(0) == b.size(0), "grouped_gemm: need one batch size per expert");
    // The reference leaves the shape of c unchecked here; a wrong one would make the
    // kernel write outside c, so it is rejected.
    TORCH_CHECK(!gate_up || (trans_b ? b.size(1) : b.size(2)) % 2 == 0,
                "grouped_gemm: with gate | up columns, b must hold an even number of them");
    const int64_t hidden_out = (trans_b ? b.size(1) : b.size(2)) / (gate_up ? 2 : 1);
    if (rows.c.defined()) {
      TORCH_CHECK(rows.c.size(0) == tokens, "grouped_gemm: c_rows needs one entry per row of the product");
      TORCH_CHECK(c.size(1) == hidden_out, "grouped_gemm: c must have hidden_out columns");
    } else {
      TORCH_CHECK(c.size(0) == tokens && c.size(1) == hidden_out,
                  "grouped_gemm: c must have shape (tokens, hidden_out)");
    }
  }

  // Transposition goes through the flags only (csrc/grouped_gemm.cu:538-540).
  TORCH_CHECK(a.is_contiguous(), "grouped_gemm: a must be contiguous");
  TORCH_CHECK(b.is_contiguous(), "grouped_gemm: b must be contiguous");
  TORCH_CHECK(c.is_contiguous(), "grouped_gemm: c must be contiguous");

  // Device-resident sizes: any number of experts (the reference stops at 512,
  // csrc/grouped_gemm.cu:120-124; here further experts go to further launches).
  if (batch_sizes.is_cuda()) {
    TORCH_CHECK(batch_sizes.is_contiguous(), "grouped_gemm: batch_sizes must be contiguous");
    if (on_device)
      TORCH_CHECK(batch_sizes.device() == a.device(), "grouped_gemm: batch_sizes is on another GPU");
  }
  if (on_device) {
    TORCH_CHECK(b.device() == a.device() && c.device() == a.device(),
                "grouped_gemm: a, b and c must be on the same GPU");
  }
}

// Workspace for the depth pieces of a call's last round (see gg_gmm): one per device and stream,
// allocated and zeroed at the first call there that can use one (gg_workspace_bytes_for) and kept
// for the life of the process.  Calls on one
// stream run one after the other, so they can share it; the kernels leave its counters zero.
torch::Tensor Workspace(const torch::Device& device, hipStream_t stream) {
  static std::mutex mu;
  static std::map<std::pair<int, hipStream_t>, torch::Tensor> cache;
  std::lock_guard<std::mutex> lock(mu);
  auto key = std::make_pair((int)device.index(), stream);
  auto it = cache.find(key);
  if (it == cache.end()) {
    torch::Tensor ws = torch::zeros({(int64_t)GG_WORKSPACE_BYTES}, torch::dtype(torch::kUInt8).device(device));
    it = cache.emplace(key, ws).first;
  }
  return it->second;
}

// One int32 word per device that the kernels OR GG_STATUS_* bits into when device-resident
// batch_sizes had to be clamped (negative, or summing past the rows of a): what a host-resident
// size vector would have been rejected for.  Read (and cleared) through size_status().
torch::Tensor SizeStatusWord(const torch::Device& device) {
  static std::mutex mu;
  static std::map<int, torch::Tensor> cache;
  std::lock_guard<std::mutex> lock(mu);
  auto it = cache.find((int)device.index());
  if (it == cache.end())
    it = cache.emplace((int)device.index(), torch::zeros({1}, torch::dtype(torch::kInt32).device(device))).first;
  return it->second;
}

void Run(const torch::Tensor& a, const torch::Tensor& b, const torch::Tensor& c, const torch::Tensor& batch_sizes,
         bool trans_a, bool trans_b, bool accumulate_f32, int64_t flags, const RowIndices& rows = RowIndices(),
         bool gate_up = false) {
  torch::Tensor sizes = batch_sizes.is_cpu() ? batch_sizes.contiguous() : batch_sizes;
  c10::hip::HIPGuardMasqueradingAsCUDA guard(a.device());
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(a.device().index()).stream();
  TORCH_CHECK(gg_init() == GG_OK, "grouped_gemm: ", gg_last_error());
  gg_gmm_args g = {};
  g.struct_bytes = sizeof(g);
  g.dtype = DtypeCode(a.scalar_type());
  g.a = a.data_ptr();
  g.b = b.data_ptr();
  g.c = c.data_ptr();
  g.batch_sizes = sizes.data_ptr<int64_t>();
  g.batch_sizes_on_device = sizes.is_cuda() ? 1 : 0;
  g.trans_a = trans_a ? 1 : 0;
  g.trans_b = trans_b ? 1 : 0;
  g.accumulate_f32 = accumulate_f32 ? 1 : 0;
  g.num_groups = sizes.size(0);
  g.tokens = rows.a.defined() ? rows.a.size(0) : a.size(0);
  g.a_row_index = rows.a.defined() ? rows.a.data_ptr<int32_t>() : nullptr;
  g.b_row_index = rows.b.defined() ? rows.b.data_ptr<int32_t>() : nullptr;
  g.c_row_index = rows.c.defined() ? rows.c.data_ptr<int32_t>() : nullptr;
  g.hidden_in = a.size(1);
  g.hidden_out = (trans_a ? b.size(1) : (trans_b ? b.size(1) : b.size(2))) / (gate_up ? 2 : 1);
  g.epilogue = gate_up ? GG_EPILOGUE_SWIGLU : GG_EPILOGUE_NONE;
  g.a_num_rows = a.size(0);
  g.c_num_rows = trans_a ? 0 : c.size(0);
  g.b_num_rows = trans_a ? (int32_t)b.size(0) : 0;
  g.flags = (int32_t)flags;
  // a workspace only for calls that can cut tiles along the depth (deep products, weight gradients)
  if (gg_workspace_bytes_for(&g) > 0) {
    torch::Tensor ws = Workspace(a.device(), stream);
    g.workspace = ws.data_ptr();
    g.workspace_bytes = (uint64_t)ws.numel();
  }
  g.stream = static_cast<void*>(stream);
  if (sizes.is_cuda()) g.size_status = SizeStatusWord(a.device()).data_ptr<int32_t>();
  const int rc = gg_gmm(&g);
  TORCH_CHECK(rc == GG_OK, "grouped_gemm: ", gg_last_error());
}

}  // namespace

void GroupedGemm(torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes,
                 bool trans_a, bool trans_b) {
  Validate(a, b, c, batch_sizes, trans_a, trans_b, /*on_device=*/true);
  Run(a, b, c, batch_sizes, trans_a, trans_b, /*accumulate_f32=*/false, /*flags=*/0);
}

// gmm with GG_FLAG_* bits, for tests that compare the ways a call can be scheduled.
void GroupedGemmWithFlags(torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes,
                          bool trans_a, bool trans_b, int64_t flags) {
  Validate(a, b, c, batch_sizes, trans_a, trans_b, /*on_device=*/true);
  Run(a, b, c, batch_sizes, trans_a, trans_b, /*accumulate_f32=*/false, flags);
}

// gmm with row indices: a gather fused into the loads of a (and of b with trans_a), a scatter
// fused into the stores of c.  An undefined (None) index leaves those rows in place.
void GroupedGemmIndexed(torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes,
                        bool trans_a, bool trans_b, c10::optional<torch::Tensor> a_rows,
                        c10::optional<torch::Tensor> b_rows, c10::optional<torch::Tensor> c_rows) {
  RowIndices rows;
  if (a_rows.has_value()) rows.a = *a_rows;
  if (b_rows.has_value()) rows.b = *b_rows;
  if (c_rows.has_value()) rows.c = *c_rows;
  Validate(a, b, c, batch_sizes, trans_a, trans_b, /*on_device=*/true, rows);
  Run(a, b, c, batch_sizes, trans_a, trans_b, /*accumulate_f32=*/false, /*flags=*/0, rows);
}

// c = silu(a @ gate) * (a @ up) with b = [gate | up] per expert, optionally with row indices.
void GroupedGemmSwiGLU(torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes, bool trans_b,
                       c10::optional<torch::Tensor> a_rows, c10::optional<torch::Tensor> c_rows) {
  RowIndices rows;
  if (a_rows.has_value()) rows.a = *a_rows;
  if (c_rows.has_value()) rows.c = *c_rows;
  Validate(a, b, c, batch_sizes, /*trans_a=*/false, trans_b, /*on_device=*/true, rows, /*gate_up=*/true);
  Run(a, b, c, batch_sizes, /*trans_a=*/false, trans_b, /*accumulate_f32=*/false, /*flags=*/0, rows, /*gate_up=*/true);
}

// c (num_experts, hidden_in, hidden_out) fp32 += per expert a_e^T @ b_e; see gg_gmm_bf16_acc_f32.
void AccumulateWeightGradient(torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes) {
  TORCH_CHECK(c.scalar_type() == torch::kFloat32, "grouped_gemm: the accumulated gradient must be float32");
  // every other check is the one of the bf16 weight-gradient call
  torch::Tensor shape_of_c = torch::empty(c.sizes(), torch::dtype(OutputType(a.scalar_type())).device(torch::kMeta));
  Validate(a, b, shape_of_c, batch_sizes, /*trans_a=*/true, /*trans_b=*/false, /*on_device=*/false);
  TORCH_CHECK(a.is_cuda() && b.is_cuda() && c.is_cuda(), "grouped_gemm: a, b and c must be GPU tensors");
  TORCH_CHECK(b.device() == a.device() && c.device() == a.device(),
              "grouped_gemm: a, b and c must be on the same GPU");
  TORCH_CHECK(c.is_contiguous(), "grouped_gemm: c must be contiguous");
  if (batch_sizes.is_cuda())
    TORCH_CHECK(batch_sizes.device() == a.device(), "grouped_gemm: batch_sizes is on another GPU");
  Run(a, b, c, batch_sizes, /*trans_a=*/true, /*trans_b=*/false, /*accumulate_f32=*/true, /*flags=*/0);
}

// GG_STATUS_* bits collected on `device` since the last call of this function (waits for the
// device): 0 unless device-resident batch_sizes had to be clamped.
int64_t SizeStatus(torch::Device device) {
  TORCH_CHECK(device.is_cuda(), "grouped_gemm: size_status is kept per GPU");
  c10::hip::HIPGuardMasqueradingAsCUDA guard(device);
  if (!device.has_index()) device = torch::Device(device.type(), c10::hip::current_device());
  torch::Tensor word = SizeStatusWord(device);
  const int64_t bits = word.item<int32_t>();
  if (bits != 0) word.zero_();
  return bits;
}

// The on-device scheduler's view of the groups, as an int64 tensor
// (num_experts, GG_SCHED_COLS) on `device`; see gg_debug_schedule.
torch::Tensor DebugSchedule(torch::Tensor batch_sizes, int64_t tokens, int64_t hidden_in,
                            int64_t hidden_out, bool trans_a, bool trans_b, torch::Device device) {
  TORCH_CHECK(batch_sizes.ndimension() == 1 && batch_sizes.scalar_type() == torch::kInt64);
  TORCH_CHECK(device.is_cuda(), "grouped_gemm: the schedule is computed on a GPU");
  torch::Tensor sizes = batch_sizes.contiguous();
  if (sizes.is_cuda()) TORCH_CHECK(sizes.device() == device);
  c10::hip::HIPGuardMasqueradingAsCUDA guard(device);
  torch::Tensor out = torch::zeros({sizes.size(0), GG_SCHED_COLS},
                                   torch::dtype(torch::kInt64).device(device));
  hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(device.index()).stream();
  const int rc = gg_debug_schedule(sizes.data_ptr<int64_t>(), sizes.is_cuda() ? 1 : 0, sizes.size(0),
                                   tokens, hidden_in, hidden_out, trans_a ? 1 : 0, trans_b ? 1 : 0,
                                   out.data_ptr<int64_t>(), static_cast<void*>(stream));
  TORCH_CHECK(rc == GG_OK, "grouped_gemm: ", gg_last_error());
  return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("gmm", &GroupedGemm, "Grouped GEMM.");
  m.def("validate",
        [](torch::Tensor a, torch::Tensor b, torch::Tensor c, torch::Tensor batch_sizes, bool trans_a,
           bool trans_b) { Validate(a, b, c, batch_sizes, trans_a, trans_b, /*on_device=*/false); },
        "Shape, rank and dtype checks of gmm without the device checks.");
  m.def("gmm_indexed", &GroupedGemmIndexed, "gmm with fused row gather / scatter.", py::arg("a"), py::arg("b"),
        py::arg("c"), py::arg("batch_sizes"), py::arg("trans_a"), py::arg("trans_b"), py::arg("a_rows") = py::none(),
        py::arg("b_rows") = py::none(), py::arg("c_rows") = py::none());
  m.def("gmm_swiglu", &GroupedGemmSwiGLU, "silu(a @ gate) * (a @ up) with b = [gate | up].", py::arg("a"),
        py::arg("b"), py::arg("c"), py::arg("batch_sizes"), py::arg("trans_b"), py::arg("a_rows") = py::none(),
        py::arg("c_rows") = py::none());
  m.def("size_status", &SizeStatus,
        "Bits collected since the last call: 1 a device-resident batch size was negative, 2 they summed past the "
        "rows of a (both clamped by the kernel).");
  m.attr("status_negative_size") = GG_STATUS_NEGATIVE_SIZE;
  m.attr("status_rows_past_end") = GG_STATUS_ROWS_PAST_END;
  m.def("gmm_with_flags", &GroupedGemmWithFlags, "gmm with GG_FLAG_* bits (testing).");
  m.attr("flag_whole_tiles") = GG_FLAG_WHOLE_TILES;
  m.attr("flag_group_order") = GG_FLAG_GROUP_ORDER;
  m.def("accumulate_weight_gradient", &AccumulateWeightGradient,
        "c (fp32) += per expert a_e^T @ b_e.");
  m.def("debug_schedule", &DebugSchedule, "Per-group table derived by the on-device scheduler.");
  m.attr("max_groups_per_launch") = GG_MAX_GROUPS_PER_LAUNCH;
  m.attr("sched_cols") = GG_SCHED_COLS;
}

}  // namespace grouped_gemm
