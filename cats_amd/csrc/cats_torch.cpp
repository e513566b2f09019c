// torch.ops.flash_gemv.* -- the op library the flash_gemv Python package loads.
//
// Same namespace, op names and positional signatures as the reference registration
// (flash_gemv/csrc/fuse_gemv_cmp.cpp:87-102), so `torch.ops.flash_gemv.<op>(...)` call sites keep working.
// Each op unpacks its tensors, checks device / dtype / contiguity / shapes, takes the current HIP stream
// and a cached workspace, and calls one entry point of the C ABI in include/cats_gemv.h.  A non-zero
// status becomes a c10::Error (the reference printf()s and exit()s: fuse_gemv_cmp_cuda.cu:2096-2097).
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <map>
#include <mutex>
#include <tuple>
#include <utility>

#include "cats_gemv.h"

namespace {

int dtype_code(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::ScalarType::Half: return CATS_F16;
    case at::ScalarType::BFloat16: return CATS_BF16;
    case at::ScalarType::Float: return CATS_F32;
    default: TORCH_CHECK(false, "flash_gemv: unsupported dtype ", t.scalar_type(), " (expected half, bfloat16 or float)");
  }
  return -1;
}

void check_status(int st, const char* op) {
  TORCH_CHECK(st == CATS_OK, "flash_gemv.", op, ": ", cats_status_string(st));
}

void check_dev(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), "flash_gemv: ", name, " must be on the GPU");
  TORCH_CHECK(t.is_contiguous(), "flash_gemv: ", name, " must be contiguous");
}

// Leading dims flattened into rows, as the reference does (fuse_gemv_cmp_cuda.cu:2339-2347).
int batch_rows(const at::Tensor& input, const char* op) {
  TORCH_CHECK(input.dim() == 2 || input.dim() == 3, "flash_gemv.", op, ": input must be (B, H) or (B, 1, H), got ", input.dim(), " dims");
  const int64_t b = input.dim() == 3 ? input.size(0) * input.size(1) : input.size(0);
  TORCH_CHECK(b >= 1 && b <= CATS_MAX_BATCH, "flash_gemv.", op, ": batch of ", b, " rows is not supported (1..", CATS_MAX_BATCH, ")");
  return (int)b;
}

void check_weight(const at::Tensor& w, const at::Tensor& like, int64_t rows, int64_t cols, const char* name) {
  check_dev(w, name);
  TORCH_CHECK(w.dim() == 2 && w.size(0) == rows && w.size(1) == cols, "flash_gemv: ", name, " must be (", rows, ", ", cols, "), got ", w.sizes());
  TORCH_CHECK(w.scalar_type() == like.scalar_type(), "flash_gemv: ", name, " dtype ", w.scalar_type(), " differs from input dtype ", like.scalar_type());
  TORCH_CHECK(w.device() == like.device(), "flash_gemv: ", name, " is on a different device than input");
}

struct Workspace {
  at::Tensor buf;
  size_t bytes = 0;
};

// One workspace per (device, stream, H, I): the carving of a workspace is tied to the layer shape, and one workspace
// serves one stream at a time.  It is allocated and zero-filled (by a kernel on the calling stream) on the first call
// for a shape; that first call must not happen under stream capture (the allocation would come out of the graph's
// private pool and the fill would be recorded into the graph), so it is refused there: run one call eagerly on the
// capturing stream first.  A captured graph keeps using the workspace of the stream it was captured on, so eager
// calls on that stream must not overlap its replays.  Entries live until the process ends (a few MB per layer shape
// and stream; torch hands out at most 32 pooled side streams per device) and the map is never destroyed: at exit the
// HIP runtime may be gone before static destructors run.
Workspace& workspace(const at::Tensor& like, int B, int H, int I, hipStream_t stream) {
  static std::mutex mu;
  static auto& cache = *new std::map<std::tuple<int, void*, int, int>, Workspace>();
  std::lock_guard<std::mutex> lock(mu);
  Workspace& ws = cache[std::make_tuple((int)like.get_device(), (void*)stream, H, I)];
  const size_t need = cats_workspace_bytes(B, H, I);
  if (ws.bytes < need) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    TORCH_CHECK(hipStreamIsCapturing(stream, &cap) == hipSuccess && cap == hipStreamCaptureStatusNone,
                "flash_gemv: the first call for a layer shape on a stream allocates its workspace and cannot run under "
                "stream capture; call the op once on this stream before capturing");
    ws.buf = at::empty({(int64_t)need}, like.options().dtype(at::kByte));
    ws.bytes = need;
    check_status(cats_workspace_init(ws.buf.data_ptr(), need, stream), "workspace_init");
  }
  return ws;
}

hipStream_t current_stream(const at::Tensor& t) { return c10::hip::getCurrentHIPStream(t.get_device()).stream(); }

// ---- the 14 reference ops -----------------------------------------------------------------------------

int64_t fuse_gemv_cmp(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& idx,
                      const double threshold) {
  check_dev(input, "input");
  const int B = batch_rows(input, "fuse_gemv_cmp");
  TORCH_CHECK(B == 1, "flash_gemv.fuse_gemv_cmp: batch must be 1");
  const int64_t H = input.size(-1), I = weight.size(0);
  check_weight(weight, input, I, H, "weight");
  check_dev(output, "output");
  check_dev(idx, "idx");
  TORCH_CHECK(output.scalar_type() == input.scalar_type() && output.numel() >= I, "flash_gemv.fuse_gemv_cmp: output must hold I values of the input dtype");
  TORCH_CHECK(idx.scalar_type() == at::kLong && idx.numel() >= I, "flash_gemv.fuse_gemv_cmp: idx must be int64 with I entries");
  hipStream_t s = current_stream(input);
  Workspace& ws = workspace(input, 1, (int)H, (int)I, s);
  int32_t* count = (int32_t*)((char*)ws.buf.data_ptr() + 768);
  check_status(cats_gate_compact(input.data_ptr(), weight.data_ptr(), output.data_ptr(), idx.data_ptr<int64_t>(), count,
                                 (int)H, (int)I, dtype_code(input), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "fuse_gemv_cmp");
  const int n = cats_read_count(count, s);
  TORCH_CHECK(n >= 0, "flash_gemv.fuse_gemv_cmp: reading the count back failed");
  return n;
}

void gate_flag_common(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag,
                      const double threshold, const char* op) {
  check_dev(input, "input");
  const int B = batch_rows(input, op);
  const int64_t H = input.size(-1), I = weight.size(0);
  check_weight(weight, input, I, H, "weight");
  check_dev(output, "output");
  check_dev(flag, "flag");
  TORCH_CHECK(output.scalar_type() == input.scalar_type() && output.numel() == B * I, "flash_gemv.", op, ": output must be (B, I) of the input dtype");
  TORCH_CHECK(flag.scalar_type() == at::kBool && flag.numel() == B * I, "flash_gemv.", op, ": flag must be bool with B*I entries");
  check_status(cats_gate_flag(input.data_ptr(), weight.data_ptr(), output.data_ptr(), (uint8_t*)flag.data_ptr(), B, (int)H,
                              (int)I, dtype_code(input), (float)threshold, current_stream(input)),
               op);
}

void fuse_gemv_flag(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag, const double threshold) {
  gate_flag_common(input, weight, output, flag, threshold, "fuse_gemv_flag");
}
void fuse_gemv_flag_batch(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag, const double threshold) {
  gate_flag_common(input, weight, output, flag, threshold, "fuse_gemv_flag_batch");
}
void fuse_gemv_flag_local(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag, const double threshold) {
  gate_flag_common(input, weight, output, flag, threshold, "fuse_gemv_flag_local");
}

void fuse_gemv_flag_gemv(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, at::Tensor& output,
                         at::Tensor& flag, const double threshold) {
  check_dev(input, "input");
  const int B = batch_rows(input, "fuse_gemv_flag_gemv");
  const int64_t H = input.size(-1), I = wgate.size(0);
  check_weight(wgate, input, I, H, "wgate");
  check_weight(wup, input, I, H, "wup");
  check_dev(output, "output");
  check_dev(flag, "flag");
  TORCH_CHECK(output.scalar_type() == input.scalar_type() && output.numel() == B * I, "flash_gemv.fuse_gemv_flag_gemv: output must be (B, I) of the input dtype");
  TORCH_CHECK(flag.scalar_type() == at::kBool && flag.numel() == B * I, "flash_gemv.fuse_gemv_flag_gemv: flag must be bool with B*I entries");
  check_status(cats_gate_up(input.data_ptr(), wgate.data_ptr(), wup.data_ptr(), output.data_ptr(), (uint8_t*)flag.data_ptr(), B,
                            (int)H, (int)I, dtype_code(input), (float)threshold, current_stream(input)),
               "fuse_gemv_flag_gemv");
}

// Whole MLP, neuron-major down weights, fp32 accumulate into `output`.
void mlp_f32_accumulate(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown,
                        at::Tensor& output, at::Tensor* flag, const double threshold, const char* op) {
  check_dev(input, "input");
  const int B = batch_rows(input, op);
  const int64_t H = input.size(-1), I = wgate.size(0);
  check_weight(wgate, input, I, H, "wgate");
  check_weight(wup, input, I, H, "wup");
  check_weight(wdown, input, I, H, "wdown (neuron-major)");
  check_dev(output, "output");
  TORCH_CHECK(output.scalar_type() == at::kFloat && output.numel() == B * H, "flash_gemv.", op, ": output must be float32 with B*H entries");
  uint8_t* fp = nullptr;
  if (flag) {
    check_dev(*flag, "flag");
    TORCH_CHECK(flag->scalar_type() == at::kBool && flag->numel() == B * I, "flash_gemv.", op, ": flag must be bool with B*I entries");
    fp = (uint8_t*)flag->data_ptr();
  }
  hipStream_t s = current_stream(input);
  Workspace& ws = workspace(input, B, (int)H, (int)I, s);
  check_status(cats_mlp(input.data_ptr(), wgate.data_ptr(), wup.data_ptr(), wdown.data_ptr(), nullptr, output.data_ptr<float>(), fp,
                        nullptr, B, (int)H, (int)I, dtype_code(input), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               op);
}

void fuse_gemv_flag_gemv_gemv(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown,
                              at::Tensor& output, at::Tensor& flag, const double threshold) {
  mlp_f32_accumulate(input, wgate, wup, wdown, output, &flag, threshold, "fuse_gemv_flag_gemv_gemv");
}
void fuse_gemv_gemv_gemv(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown,
                         at::Tensor& output, const double threshold) {
  mlp_f32_accumulate(input, wgate, wup, wdown, output, nullptr, threshold, "fuse_gemv_gemv_gemv");
}
void flag_gemv_gemv_atomic(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown,
                           at::Tensor& output, const double threshold) {
  mlp_f32_accumulate(input, wgate, wup, wdown, output, nullptr, threshold, "flag_gemv_gemv_atomic");
}

void fuse_flag_gemv_local(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag) {
  check_dev(input, "input");
  const int B = batch_rows(input, "fuse_flag_gemv_local");
  const int64_t H = input.size(-1), I = weight.size(0);
  check_weight(weight, input, I, H, "weight");
  check_dev(output, "output");
  check_dev(flag, "flag");
  TORCH_CHECK(output.scalar_type() == input.scalar_type() && output.numel() == B * I, "flash_gemv.fuse_flag_gemv_local: output must be (B, I) of the input dtype");
  TORCH_CHECK(flag.scalar_type() == at::kBool && flag.numel() == B * I, "flash_gemv.fuse_flag_gemv_local: flag must be bool with B*I entries");
  check_status(cats_up_flag(input.data_ptr(), weight.data_ptr(), output.data_ptr(), (const uint8_t*)flag.data_ptr(), output.data_ptr(), 0,
                            B, (int)H, (int)I, dtype_code(input), current_stream(input)),
               "fuse_flag_gemv_local");
}

void atomic_gemv(const at::Tensor& input, const at::Tensor& weight, at::Tensor& output, at::Tensor& flag) {
  check_dev(input, "input");
  const int B = batch_rows(input, "atomic_gemv");
  const int64_t I = input.size(-1), H = weight.size(1);
  check_weight(weight, input, I, H, "weight (neuron-major)");
  check_dev(output, "output");
  check_dev(flag, "flag");
  TORCH_CHECK(output.scalar_type() == at::kFloat && output.numel() == B * H, "flash_gemv.atomic_gemv: output must be float32 with B*H entries");
  TORCH_CHECK(flag.scalar_type() == at::kBool && flag.numel() == B * I, "flash_gemv.atomic_gemv: flag must be bool with B*I entries");
  hipStream_t s = current_stream(input);
  Workspace& ws = workspace(input, B, (int)H, (int)I, s);
  check_status(cats_down_flag(input.data_ptr(), weight.data_ptr(), (const uint8_t*)flag.data_ptr(), output.data_ptr<float>(), nullptr, B,
                              (int)H, (int)I, dtype_code(input), ws.buf.data_ptr(), ws.bytes, s),
               "atomic_gemv");
}

void mlp_rowmajor(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown, at::Tensor& output,
                  const double threshold, const char* op) {
  check_dev(input, "input");
  const int B = batch_rows(input, op);
  const int64_t H = input.size(-1), I = wgate.size(0);
  check_weight(wgate, input, I, H, "wgate");
  check_weight(wup, input, I, H, "wup");
  check_weight(wdown, input, H, I, "wdown");
  check_dev(output, "output");
  TORCH_CHECK(output.scalar_type() == input.scalar_type() && output.numel() == B * H, "flash_gemv.", op, ": output must be (B, H) of the input dtype");
  hipStream_t s = current_stream(input);
  Workspace& ws = workspace(input, B, (int)H, (int)I, s);
  check_status(cats_mlp_rowmajor_down(input.data_ptr(), wgate.data_ptr(), wup.data_ptr(), wdown.data_ptr(), output.data_ptr(), B, (int)H,
                                      (int)I, dtype_code(input), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               op);
}

void flag_gemv_gemv(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown, at::Tensor& output,
                    const double threshold) {
  mlp_rowmajor(input, wgate, wup, wdown, output, threshold, "flag_gemv_gemv");
}

at::Tensor inner_common(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown,
                        const double threshold, at::ScalarType want, const char* op) {
  TORCH_CHECK(input.scalar_type() == want, "flash_gemv.", op, ": input must be ", want, ", got ", input.scalar_type());
  at::Tensor output = at::empty(input.sizes(), input.options());
  mlp_rowmajor(input, wgate, wup, wdown, output, threshold, op);
  return output;
}
at::Tensor flag_gemv_gemv_inner(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown, const double threshold) {
  return inner_common(input, wgate, wup, wdown, threshold, at::kHalf, "flag_gemv_gemv_inner");
}
at::Tensor flag_gemv_gemv_inner_fp32(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown, const double threshold) {
  return inner_common(input, wgate, wup, wdown, threshold, at::kFloat, "flag_gemv_gemv_inner_fp32");
}
at::Tensor flag_gemv_gemv_inner_bf16(const at::Tensor& input, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown, const double threshold) {
  return inner_common(input, wgate, wup, wdown, threshold, at::kBFloat16, "flag_gemv_gemv_inner_bf16");
}

// ---- ops behind the Python composites (the reference runs Triton there: flash_gemv/flash_gemv/kernels.py) ---

// gather_gemv_elemul_flag_3d: x (B,1,H), x_1 (B,1,I), wup (I,H), flags (B,1,I) bool -> (B,1,I) in x.dtype
at::Tensor cats_up_flag_op(const at::Tensor& x, const at::Tensor& x_1, const at::Tensor& wup, const at::Tensor& flags) {
  check_dev(x, "x");
  const int B = batch_rows(x, "cats_up_flag");
  const int64_t H = x.size(-1), I = wup.size(0);
  check_weight(wup, x, I, H, "wup");
  check_dev(x_1, "x_1");
  check_dev(flags, "flags");
  TORCH_CHECK(x_1.scalar_type() == x.scalar_type() && x_1.numel() == B * I, "flash_gemv.cats_up_flag: x_1 must be (B, I) of x's dtype");
  TORCH_CHECK(flags.scalar_type() == at::kBool && flags.numel() == B * I, "flash_gemv.cats_up_flag: flags must be bool with B*I entries");
  at::Tensor out = at::empty_like(x_1);
  check_status(cats_up_flag(x.data_ptr(), wup.data_ptr(), x_1.data_ptr(), (const uint8_t*)flags.data_ptr(), out.data_ptr(), 0, B, (int)H,
                            (int)I, dtype_code(x), current_stream(x)),
               "cats_up_flag");
  return out;
}

// gather_transposed_gemv_flag_3d: x (B,1,I), weight (I,H) neuron-major, flags (B,1,I) -> (B,1,H) in weight.dtype
at::Tensor cats_down_flag_op(const at::Tensor& x, const at::Tensor& weight, const at::Tensor& flags) {
  check_dev(x, "x");
  const int B = batch_rows(x, "cats_down_flag");
  const int64_t I = weight.size(0), H = weight.size(1);
  check_weight(weight, x, I, H, "weight (neuron-major)");
  check_dev(flags, "flags");
  TORCH_CHECK(x.size(-1) == I, "flash_gemv.cats_down_flag: x must have I columns");
  TORCH_CHECK(flags.scalar_type() == at::kBool && flags.numel() == B * I, "flash_gemv.cats_down_flag: flags must be bool with B*I entries");
  std::vector<int64_t> shape(x.sizes().begin(), x.sizes().end());
  shape.back() = H;
  at::Tensor out = at::empty(shape, weight.options());
  hipStream_t s = current_stream(x);
  Workspace& ws = workspace(x, B, (int)H, (int)I, s);
  check_status(cats_down_flag(x.data_ptr(), weight.data_ptr(), (const uint8_t*)flags.data_ptr(), nullptr, out.data_ptr(), B, (int)H, (int)I,
                              dtype_code(x), ws.buf.data_ptr(), ws.bytes, s),
               "cats_down_flag");
  return out;
}

// gather_gemv / gather_gemv_elemul_indirect_index_2d: x (B, H), weight (Z, H), idx (M,) int64 -> (B, M)
at::Tensor cats_up_index_op(const at::Tensor& x, const at::Tensor& weight, const at::Tensor& idx, const c10::optional<at::Tensor>& bias,
                            const c10::optional<at::Tensor>& scale, int64_t activation) {
  check_dev(x, "x");
  TORCH_CHECK(x.dim() == 2, "flash_gemv.cats_up_index: x must be (batch, N)");
  const int64_t B = x.size(0), H = x.size(1), Z = weight.size(0), M = idx.numel();
  TORCH_CHECK(B >= 1 && B <= 8, "flash_gemv.cats_up_index: batch of ", B, " rows is not supported (1..8)");
  check_weight(weight, x, Z, H, "weight");
  check_dev(idx, "idx");
  TORCH_CHECK(idx.scalar_type() == at::kLong && idx.dim() == 1, "flash_gemv.cats_up_index: idx must be a 1-D int64 tensor");
  const void* bp = nullptr;
  const void* sp = nullptr;
  if (bias.has_value() && bias->defined()) {
    check_dev(*bias, "bias");
    TORCH_CHECK(bias->scalar_type() == x.scalar_type() && bias->numel() == Z, "flash_gemv.cats_up_index: bias must be (Z,) of x's dtype");
    bp = bias->data_ptr();
  }
  if (scale.has_value() && scale->defined()) {
    check_dev(*scale, "scale");
    TORCH_CHECK(scale->scalar_type() == x.scalar_type() && scale->numel() == M, "flash_gemv.cats_up_index: scale must have one entry per index, in x's dtype");
    sp = scale->data_ptr();
  }
  at::Tensor out = at::empty({B, M}, x.options());
  check_status(cats_up_index(x.data_ptr(), weight.data_ptr(), idx.data_ptr<int64_t>(), (int)M, bp, sp, (int)activation, out.data_ptr(), (int)B,
                             (int)H, (int)Z, dtype_code(x), current_stream(x)),
               "cats_up_index");
  return out;
}

// gather_transposed_gemv / gather_transposed_gemv_indirect_index_2d: z (B, M), weight (Z, N) neuron-major, idx (M,) -> (B, N)
at::Tensor cats_down_index_op(const at::Tensor& z, const at::Tensor& weight, const at::Tensor& idx, const c10::optional<at::Tensor>& bias) {
  check_dev(z, "x");
  TORCH_CHECK(z.dim() == 2, "flash_gemv.cats_down_index: x must be (batch, M)");
  const int64_t B = z.size(0), M = z.size(1), Z = weight.size(0), H = weight.size(1);
  TORCH_CHECK(B >= 1 && B <= 8, "flash_gemv.cats_down_index: batch of ", B, " rows is not supported (1..8)");
  check_weight(weight, z, Z, H, "weight (neuron-major)");
  check_dev(idx, "idx");
  TORCH_CHECK(idx.scalar_type() == at::kLong && idx.dim() == 1 && idx.numel() == M, "flash_gemv.cats_down_index: idx must be int64 with one entry per column of x");
  const void* bp = nullptr;
  if (bias.has_value() && bias->defined()) {
    check_dev(*bias, "bias");
    TORCH_CHECK(bias->scalar_type() == z.scalar_type() && bias->numel() == H, "flash_gemv.cats_down_index: bias must be (N,) of x's dtype");
    bp = bias->data_ptr();
  }
  at::Tensor out = at::empty({B, H}, z.options());
  hipStream_t s = current_stream(z);
  Workspace& ws = workspace(z, (int)B, (int)H, (int)Z, s);
  check_status(cats_down_index(z.data_ptr(), weight.data_ptr(), idx.data_ptr<int64_t>(), (int)M, bp, out.data_ptr(), (int)B, (int)H, (int)Z,
                               dtype_code(z), ws.buf.data_ptr(), ws.bytes, s),
               "cats_down_index");
  return out;
}

// Whole CATS MLP in two launches: x (B,1,H) or (B,H); wgate, wup, wdown_t all (I,H).  Returns x-shaped y.
at::Tensor cats_mlp_op(const at::Tensor& x, const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown_t, const double threshold) {
  check_dev(x, "x");
  const int B = batch_rows(x, "cats_mlp");
  const int64_t H = x.size(-1), I = wgate.size(0);
  check_weight(wgate, x, I, H, "wgate");
  check_weight(wup, x, I, H, "wup");
  check_weight(wdown_t, x, I, H, "wdown_t (neuron-major)");
  at::Tensor out = at::empty_like(x);
  hipStream_t s = current_stream(x);
  Workspace& ws = workspace(x, B, (int)H, (int)I, s);
  check_status(cats_mlp(x.data_ptr(), wgate.data_ptr(), wup.data_ptr(), wdown_t.data_ptr(), out.data_ptr(), nullptr, nullptr, nullptr, B, (int)H,
                        (int)I, dtype_code(x), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "cats_mlp");
  return out;
}

// Sparse up + sparse down given the gate activations x_1 (gemv_gemv_triton of the reference package).
at::Tensor cats_up_down_op(const at::Tensor& x, const at::Tensor& x_1, const at::Tensor& wup, const at::Tensor& wdown_t, const double threshold) {
  check_dev(x, "x");
  check_dev(x_1, "x_1");
  const int B = batch_rows(x, "cats_up_down");
  const int64_t H = x.size(-1), I = wup.size(0);
  check_weight(wup, x, I, H, "wup");
  check_weight(wdown_t, x, I, H, "wdown_t (neuron-major)");
  TORCH_CHECK(x_1.scalar_type() == x.scalar_type() && x_1.numel() == (int64_t)B * I, "flash_gemv.cats_up_down: x_1 must hold B*I gate activations of x's dtype");
  at::Tensor out = at::empty_like(x);
  hipStream_t s = current_stream(x);
  Workspace& ws = workspace(x, B, (int)H, (int)I, s);
  check_status(cats_up_down(x.data_ptr(), x_1.data_ptr(), wup.data_ptr(), wdown_t.data_ptr(), out.data_ptr(), B, (int)H, (int)I, dtype_code(x),
                            (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "cats_up_down");
  return out;
}

// out = h + MLP(norm_weight * rms_norm(h, eps)): the tail of a decoder layer in two launches.
at::Tensor cats_mlp_norm_residual_op(const at::Tensor& h, const at::Tensor& norm_weight, const double eps, const at::Tensor& wgate,
                                     const at::Tensor& wup, const at::Tensor& wdown_t, const double threshold) {
  check_dev(h, "h");
  const int B = batch_rows(h, "cats_mlp_norm_residual");
  const int64_t H = h.size(-1), I = wgate.size(0);
  check_weight(wgate, h, I, H, "wgate");
  check_weight(wup, h, I, H, "wup");
  check_weight(wdown_t, h, I, H, "wdown_t (neuron-major)");
  TORCH_CHECK(norm_weight.is_cuda() && norm_weight.is_contiguous() && norm_weight.scalar_type() == h.scalar_type() &&
                  norm_weight.numel() == H && norm_weight.get_device() == h.get_device(),
              "flash_gemv.cats_mlp_norm_residual: norm_weight must be a contiguous (H,) tensor of h's dtype on h's device");
  at::Tensor out = at::empty_like(h);
  hipStream_t s = current_stream(h);
  Workspace& ws = workspace(h, B, (int)H, (int)I, s);
  check_status(cats_mlp_norm_residual(h.data_ptr(), norm_weight.data_ptr(), (float)eps, wgate.data_ptr(), wup.data_ptr(), wdown_t.data_ptr(),
                                      out.data_ptr(), B, (int)H, (int)I, dtype_code(h), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "cats_mlp_norm_residual");
  return out;
}

// (out, next) with out as above and next = next_norm_weight * rms_norm(out, next_eps): the norm the following layer starts with.
std::tuple<at::Tensor, at::Tensor> cats_mlp_norm_residual_norm_op(const at::Tensor& h, const at::Tensor& norm_weight, const double eps,
                                                                  const at::Tensor& wgate, const at::Tensor& wup, const at::Tensor& wdown_t,
                                                                  const double threshold, const at::Tensor& next_norm_weight,
                                                                  const double next_eps) {
  check_dev(h, "h");
  const int B = batch_rows(h, "cats_mlp_norm_residual_norm");
  const int64_t H = h.size(-1), I = wgate.size(0);
  check_weight(wgate, h, I, H, "wgate");
  check_weight(wup, h, I, H, "wup");
  check_weight(wdown_t, h, I, H, "wdown_t (neuron-major)");
  for (const at::Tensor* w : {&norm_weight, &next_norm_weight})
    TORCH_CHECK(w->is_cuda() && w->is_contiguous() && w->scalar_type() == h.scalar_type() && w->numel() == H &&
                    w->get_device() == h.get_device(),
                "flash_gemv.cats_mlp_norm_residual_norm: the norm weights must be contiguous (H,) tensors of h's dtype on h's device");
  at::Tensor out = at::empty_like(h);
  at::Tensor next = at::empty_like(h);
  hipStream_t s = current_stream(h);
  Workspace& ws = workspace(h, B, (int)H, (int)I, s);
  check_status(cats_mlp_norm_residual_norm(h.data_ptr(), norm_weight.data_ptr(), (float)eps, wgate.data_ptr(), wup.data_ptr(),
                                           wdown_t.data_ptr(), out.data_ptr(), next_norm_weight.data_ptr(), (float)next_eps, next.data_ptr(),
                                           B, (int)H, (int)I, dtype_code(h), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "cats_mlp_norm_residual_norm");
  return {out, next};
}

// Same, also returning the per-row flags (B*I bool) and the number of neurons fetched (int32 scalar tensor).
std::tuple<at::Tensor, at::Tensor, at::Tensor> cats_mlp_stats_op(const at::Tensor& x, const at::Tensor& wgate, const at::Tensor& wup,
                                                                 const at::Tensor& wdown_t, const double threshold) {
  check_dev(x, "x");
  const int B = batch_rows(x, "cats_mlp_stats");
  const int64_t H = x.size(-1), I = wgate.size(0);
  check_weight(wgate, x, I, H, "wgate");
  check_weight(wup, x, I, H, "wup");
  check_weight(wdown_t, x, I, H, "wdown_t (neuron-major)");
  at::Tensor out = at::empty_like(x);
  at::Tensor flags = at::empty({B, I}, x.options().dtype(at::kBool));
  at::Tensor count = at::empty({}, x.options().dtype(at::kInt));
  hipStream_t s = current_stream(x);
  Workspace& ws = workspace(x, B, (int)H, (int)I, s);
  check_status(cats_mlp(x.data_ptr(), wgate.data_ptr(), wup.data_ptr(), wdown_t.data_ptr(), out.data_ptr(), nullptr, (uint8_t*)flags.data_ptr(),
                        count.data_ptr<int32_t>(), B, (int)H, (int)I, dtype_code(x), (float)threshold, ws.buf.data_ptr(), ws.bytes, s),
               "cats_mlp_stats");
  return {out, flags, count};
}

}  // namespace

TORCH_LIBRARY(flash_gemv, m) {
  m.def("fuse_gemv_cmp", fuse_gemv_cmp);
  m.def("fuse_gemv_flag", fuse_gemv_flag);
  m.def("fuse_gemv_flag_gemv", fuse_gemv_flag_gemv);
  m.def("fuse_gemv_flag_gemv_gemv", fuse_gemv_flag_gemv_gemv);
  m.def("fuse_gemv_gemv_gemv", fuse_gemv_gemv_gemv);
  m.def("fuse_gemv_flag_batch", fuse_gemv_flag_batch);
  m.def("fuse_gemv_flag_local", fuse_gemv_flag_local);
  m.def("fuse_flag_gemv_local", fuse_flag_gemv_local);
  m.def("atomic_gemv", atomic_gemv);
  m.def("flag_gemv_gemv_atomic", flag_gemv_gemv_atomic);
  m.def("flag_gemv_gemv", flag_gemv_gemv);
  m.def("flag_gemv_gemv_inner", flag_gemv_gemv_inner);
  m.def("flag_gemv_gemv_inner_fp32", flag_gemv_gemv_inner_fp32);
  m.def("flag_gemv_gemv_inner_bf16", flag_gemv_gemv_inner_bf16);
  // HIP replacements for the Triton wrappers and the fused two-launch MLP
  m.def("cats_up_flag", cats_up_flag_op);
  m.def("cats_down_flag", cats_down_flag_op);
  m.def("cats_up_index", cats_up_index_op);
  m.def("cats_down_index", cats_down_index_op);
  m.def("cats_mlp", cats_mlp_op);
  m.def("cats_mlp_norm_residual", cats_mlp_norm_residual_op);
  m.def("cats_mlp_norm_residual_norm", cats_mlp_norm_residual_norm_op);
  m.def("cats_up_down", cats_up_down_op);
  m.def("cats_mlp_stats", cats_mlp_stats_op);
}
