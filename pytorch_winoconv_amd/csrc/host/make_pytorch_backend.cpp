// MakePytorchBackend: the compiled extension module of the reference (pybind/bind.cpp:10-24,
// pybind/extern.hpp:1-9) re-built over libwinoconv_hip.so.  Same names, same positional signatures:
// Foo, AddGPU, WinoSplit, WinoConcat, DWM - plus the two entry points named after the reference's
// source files, winograd_conv (src/winograd_conv.cpp) and split_and_concat (src/split_and_concat.cpp).
//
// This file is plain C++ (g++, no device code): it checks devices, dtypes, shapes and contiguity,
// takes scratch memory from torch's caching allocator and the stream from torch's current HIP
// stream, releases the GIL, and calls the C ABI of include/winoconv.h.  Errors become Python
// exceptions (the reference prints and calls exit(-1): src/winograd_conv.cpp:80-84,116-126).
// Wider than the reference: float16 and bfloat16 are dispatched by tensor dtype (the reference binds
// float only: bind.cpp:19-23), stride 2 and every kernel extent 1..10 work.
#include <torch/extension.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>

#include <optional>
#include <sstream>
#include <stdexcept>
#include <string>
#include <thread>
#include <vector>

#include "../../../include/winoconv.h"

namespace py = pybind11;

namespace {

struct Unsupported : std::runtime_error { using std::runtime_error::runtime_error; };
struct WinoconvError : std::runtime_error { using std::runtime_error::runtime_error; };

// wc_status -> C++ exception (translated to ValueError / NotImplementedError / WinoconvError below)
void check(int rc) {
  if (rc == WC_OK) return;
  const std::string msg = wc_last_error();
  if (rc == WC_ERR_BAD_ARG) throw std::invalid_argument(msg);
  if (rc == WC_ERR_UNSUPPORTED) throw Unsupported(msg);
  throw WinoconvError("winoconv error " + std::to_string(rc) + ": " + msg);
}

int dtype_of(const at::Tensor& t) {
  switch (t.scalar_type()) {
    case at::kFloat: return WC_F32;
    case at::kHalf: return WC_F16;
    case at::kBFloat16: return WC_BF16;
    default: {
      std::ostringstream os;
      os << "winoconv supports float32, float16 and bfloat16, got " << t.scalar_type();
      throw py::type_error(os.str());
    }
  }
}

void require_gpu(const at::Tensor& t, const char* what) {
  if (!t.is_cuda()) {
    std::ostringstream os;
    os << what << ": winoconv runs on the GPU only: got a " << t.device() << " tensor";
    throw std::invalid_argument(os.str());
  }
  dtype_of(t);
}

void* stream_of(const at::Tensor& t) {
  return c10::hip::getCurrentHIPStream(t.device().index()).stream();
}

// Workspace of a call.  Small ones (the filter of a one-kernel layer: a few hundred KB, where the 1.6 us of an
// allocation is a visible part of a 10 us call) are kept per thread, device and stream: calls on one stream
// run in order, so the next call may write where the last one read.  A thread keeps at most kKeptSlots of them
// (4 MB): a further (device, stream) pair takes the slot used longest ago, whose tensor goes back to the caching
// allocator, which hands a block to later allocations of the stream it was allocated on only, in stream order.
// A thread that ends returns its workspaces; the thread that imported the module keeps them until the process ends
// (its thread-local objects are destroyed during exit(), when the interpreter has already been finalised).
// A stream under capture gets a fresh allocation from the graph's own pool instead.
const std::thread::id g_import_thread = std::this_thread::get_id();

struct KeptWorkspaces {
  struct Kept { int device; void* stream; at::Tensor ws; uint64_t used; };
  std::vector<Kept> slots;
  uint64_t clock = 0;
  ~KeptWorkspaces() {
    if (std::this_thread::get_id() == g_import_thread) new std::vector<Kept>(std::move(slots));   // never freed
  }
};

at::Tensor workspace_for(const at::Tensor& like, size_t bytes, void* stream) {
  constexpr size_t kKept = 1u << 20;
  constexpr size_t kKeptSlots = 4;
  auto fresh = [&](size_t n) { return at::empty({(int64_t)n}, like.options().dtype(at::kByte)); };
  if (bytes > kKept) return fresh(bytes);
  if (stream != nullptr) {                      // the default stream cannot be captured
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(static_cast<hipStream_t>(stream), &capturing) != hipSuccess ||
        capturing != hipStreamCaptureStatusNone)
      return fresh(bytes);
  }
  thread_local KeptWorkspaces kept;
  const int device = like.device().index();
  for (auto& k : kept.slots)
    if (k.device == device && k.stream == stream) {
      k.used = ++kept.clock;
      return k.ws;
    }
  if (kept.slots.size() < kKeptSlots) {
    kept.slots.push_back(KeptWorkspaces::Kept{device, stream, fresh(kKept), ++kept.clock});
    return kept.slots.back().ws;
  }
  auto* oldest = &kept.slots[0];
  for (auto& k : kept.slots)
    if (k.used < oldest->used) oldest = &k;
  *oldest = KeptWorkspaces::Kept{device, stream, fresh(kKept), ++kept.clock};
  return oldest->ws;
}

std::string shape_str(at::IntArrayRef s) {
  std::ostringstream os;
  os << "(";
  for (size_t i = 0; i < s.size(); ++i) os << (i ? ", " : "") << s[i];
  os << ")";
  return os.str();
}

void check_out(const at::Tensor& out, const std::vector<int64_t>& shape, const at::Tensor& like, const char* what) {
  if (out.sizes().vec() != shape || out.scalar_type() != like.scalar_type() || out.device() != like.device() ||
      !out.is_contiguous()) {
    std::ostringstream os;
    os << what << ": output must be a contiguous " << like.scalar_type() << " tensor of shape " << shape_str(shape)
       << " on " << like.device() << ", got " << shape_str(out.sizes());
    throw std::invalid_argument(os.str());
  }
}

// ---- template demo of the reference (src/foo.cpp, src/add.cpp:9-31), kept importable -----------------------
class Foo {
 public:
  void setKey(int key) { key_ = key; }
  int getKey() const { return key_; }
  std::string toString() const { return "< Foo, key: " + std::to_string(key_) + " > "; }
 private:
  int key_ = 0;
};

void AddGPU(at::Tensor in_a, at::Tensor in_b, at::Tensor out_c) {
  if (in_a.numel() != in_b.numel())
    throw std::invalid_argument("AddGPU: inputs must have the same number of elements");   // src/add.cpp:14-17
  out_c.resize_(in_a.sizes());
  at::add_out(out_c, in_a, in_b.view_as(in_a));
}

// ---- tile copies (src/split_and_concat.cpp:14-76) ---------------------------------------------------------------
void WinoSplit(at::Tensor in_a, at::Tensor out, int block_D, int block_H, int block_W, int output_block_size,
               int nD, int nH, int nW, bool two_dimension) {
  require_gpu(in_a, "WinoSplit");
  require_gpu(out, "WinoSplit");
  if (!in_a.is_contiguous()) throw std::invalid_argument("WinoSplit: in_a must be contiguous channel-last");
  if (in_a.dim() != (two_dimension ? 4 : 5))
    throw std::invalid_argument("WinoSplit: in_a must be (B, H, W, C) or (B, D, H, W, C), got " + shape_str(in_a.sizes()));
  const int es = (int)in_a.element_size(), m = output_block_size;
  void* st = stream_of(in_a);
  if (two_dimension) {
    const int B = in_a.size(0), H = in_a.size(1), W = in_a.size(2), C = in_a.size(3);
    check_out(out, {(int64_t)B * nH * nW, C, block_H, block_W}, in_a, "WinoSplit");
    py::gil_scoped_release nogil;
    check(wc_wino_split2d(in_a.data_ptr(), out.data_ptr(), B, H, W, C, block_H, block_W, m, nH, nW, es, st));
  } else {
    const int B = in_a.size(0), D = in_a.size(1), H = in_a.size(2), W = in_a.size(3), C = in_a.size(4);
    check_out(out, {(int64_t)B * nD * nH * nW, C, block_D, block_H, block_W}, in_a, "WinoSplit");
    py::gil_scoped_release nogil;
    check(wc_wino_split3d(in_a.data_ptr(), out.data_ptr(), B, D, H, W, C, block_D, block_H, block_W, m, nD, nH, nW,
                          es, st));
  }
}

// Like the reference (src/split_and_concat.cpp:44-76), the output extents are read from `out` and B follows
// from the tile count.
void WinoConcat(at::Tensor in_a, at::Tensor out, int output_block_size, bool two_dimension) {
  require_gpu(in_a, "WinoConcat");
  require_gpu(out, "WinoConcat");
  if (!in_a.is_contiguous() || !out.is_contiguous()) throw std::invalid_argument("WinoConcat: tensors must be contiguous");
  const int nd = two_dimension ? 2 : 3, m = output_block_size;
  if (in_a.dim() != nd + 2 || out.dim() != nd + 2 || m < 1)
    throw std::invalid_argument("WinoConcat: expected tiles (N, K, [m,] m, m) and a channel-last output");
  const int64_t N = in_a.size(0), K = in_a.size(1);
  int64_t per = 1;
  for (int a = 0; a < nd; ++a) per *= (out.size(1 + a) + m - 1) / m;
  const int64_t B = per ? N / per : 0;
  if (B * per != N || out.size(0) != B || out.size(nd + 1) != K || out.scalar_type() != in_a.scalar_type()) {
    std::ostringstream os;
    os << "WinoConcat: " << N << " tiles of " << K << " channels do not fill an output of shape " << shape_str(out.sizes());
    throw std::invalid_argument(os.str());
  }
  const int es = (int)in_a.element_size();
  void* st = stream_of(in_a);
  py::gil_scoped_release nogil;
  if (two_dimension)
    check(wc_wino_concat2d(in_a.data_ptr(), out.data_ptr(), (int)B, (int)out.size(1), (int)out.size(2), (int)K, m, es, st));
  else
    check(wc_wino_concat3d(in_a.data_ptr(), out.data_ptr(), (int)B, (int)out.size(1), (int)out.size(2), (int)out.size(3),
                           (int)K, m, es, st));
}

void split_and_concat(const std::string& direction, at::Tensor in_a, at::Tensor out, py::args args) {
  if (direction == "split") {
    if (args.size() != 8) throw std::invalid_argument("split_and_concat('split', in_a, out, block_D, block_H, block_W, "
                                                      "output_block_size, nD, nH, nW, two_dimension)");
    WinoSplit(in_a, out, args[0].cast<int>(), args[1].cast<int>(), args[2].cast<int>(), args[3].cast<int>(),
              args[4].cast<int>(), args[5].cast<int>(), args[6].cast<int>(), args[7].cast<bool>());
  } else if (direction == "concat") {
    if (args.size() != 2) throw std::invalid_argument("split_and_concat('concat', in_a, out, output_block_size, two_dimension)");
    WinoConcat(in_a, out, args[0].cast<int>(), args[1].cast<bool>());
  } else {
    throw std::invalid_argument("split_and_concat: direction must be 'split' or 'concat'");
  }
}

// ---- whole convolution (src/winograd_conv.cpp:17-127) -----------------------------------------------------------------
// Input (B, D, H, W, C) contiguous; Weight any strided view with dims (kD, kH, kW, C, K) (the reference's
// layout, dwm.py:85,133); Output (B, oD, oH, oW, K) contiguous; a 2-D problem has D = kD = 1.  Returns the
// output tile really used (wc_conv_auto may replace 4 by 3 or 2).
int winograd_conv(at::Tensor Input, at::Tensor Weight, at::Tensor Output, std::optional<at::Tensor> bias, int stride,
                  py::object padding, int m, const std::string& algo, std::optional<at::Tensor> U, int chunk_images,
                  py::object stacked) {
  if (algo != "dwm" && algo != "whole") throw std::invalid_argument("winograd_conv: algo must be 'dwm' or 'whole', got '" + algo + "'");
  if (Input.dim() != 5 || Weight.dim() != 5 || Output.dim() != 5)
    throw std::invalid_argument("winograd_conv: expected 5-D channel-last Input/Output and a 5-D Weight");
  const int64_t K = Weight.size(4), C = Weight.size(3);
  if (bias && bias->defined()) {
    if (bias->dim() != 1 || bias->numel() != K)
      throw std::invalid_argument("bias must be a 1-D tensor of " + std::to_string(K) + " values (one per output channel), got shape " +
                                  shape_str(bias->sizes()));
    if (bias->scalar_type() != Input.scalar_type()) *bias = bias->to(Input.scalar_type());
    if (bias->device() != Input.device()) throw std::invalid_argument("bias and Input are on different devices");
    *bias = bias->contiguous();
  }
  if (U && U->defined()) {
    if (U->scalar_type() != Input.scalar_type()) {
      std::ostringstream os;
      os << "the transformed filter is " << U->scalar_type() << ", the input is " << Input.scalar_type()
         << ": transform the filter in the input's dtype";
      throw py::type_error(os.str());
    }
    if (U->device() != Input.device()) throw std::invalid_argument("the transformed filter and Input are on different devices");
  }
  require_gpu(Input, "winograd_conv");
  require_gpu(Weight, "winograd_conv");
  require_gpu(Output, "winograd_conv");
  if (!Input.is_contiguous() || !Output.is_contiguous()) throw std::invalid_argument("winograd_conv: Input and Output must be contiguous");
  if (Weight.scalar_type() != Input.scalar_type() || Output.scalar_type() != Input.scalar_type())
    throw py::type_error("winograd_conv: Input, Weight and Output must share one dtype");
  if (Input.size(4) != C)
    throw std::invalid_argument("winograd_conv: Input has " + std::to_string(Input.size(4)) + " channels, Weight expects " + std::to_string(C));

  wc_conv_desc d{};
  const bool flat = Input.size(1) == 1 && Weight.size(0) == 1;
  d.ndim = flat ? 2 : 3;
  d.N = (int)Input.size(0); d.C = (int)C; d.K = (int)K;
  for (int a = 0; a < 3; ++a) { d.in[a] = (int)Input.size(1 + a); d.kernel[a] = (int)Weight.size(a); }
  if (py::isinstance<py::int_>(padding)) {
    const int p = padding.cast<int>();
    d.pad[0] = flat ? 0 : p; d.pad[1] = p; d.pad[2] = p;
  } else {
    const auto p = padding.cast<std::vector<int>>();
    if (p.size() != 3) throw std::invalid_argument("winograd_conv: padding is one int or (pD, pH, pW)");
    for (int a = 0; a < 3; ++a) d.pad[a] = p[a];
  }
  d.stride = stride; d.m = m; d.dtype = dtype_of(Input);
  d.chunk_images = chunk_images;
  d.whole_kernel = algo == "whole";
  d.stacked = stacked.is_none() ? -1 : (py::isinstance<py::bool_>(stacked) ? (int)stacked.cast<bool>() : stacked.cast<int>());
  if (d.stacked > 2 || d.stacked < -1) throw std::invalid_argument("winograd_conv: stacked is None, False, True or 2");
  // the one-kernel path of thin layers wants 16-byte aligned operands; a legal view can start anywhere
  auto misaligned = [](const at::Tensor& t) { return (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15) != 0; };
  d.unfused = misaligned(Input) || misaligned(Output) || (U && U->defined() && misaligned(*U));
  check(wc_conv_auto(&d));
  int out[3], grid[3];
  check(wc_conv_out_dims(&d, out, grid));
  check_out(Output, {d.N, out[0], out[1], out[2], d.K}, Input, "winograd_conv");
  if (U && U->defined()) {
    size_t ue = 0;
    check(wc_conv_u_elems(&d, &ue));
    if (!U->is_contiguous() || (size_t)U->numel() != ue)
      throw std::invalid_argument("U has " + std::to_string(U->numel()) + " elements, this convolution needs a contiguous transformed "
                                  "filter of " + std::to_string(ue) + " (transform_filter must be called with the same options)");
  }
  size_t bytes = 0;
  check(wc_conv_workspace_bytes(&d, &bytes));
  at::Tensor ws = at::empty({(int64_t)bytes}, Input.options().dtype(at::kByte));        // torch's caching allocator
  // Weight is (kD, kH, kW, C, K): its strides in (K, C, kD, kH, kW) order, no copy
  const int64_t s[5] = {Weight.stride(4), Weight.stride(3), Weight.stride(0), Weight.stride(1), Weight.stride(2)};
  void* st = stream_of(Input);
  const void* bp = bias && bias->defined() ? bias->data_ptr() : nullptr;
  const void* up = U && U->defined() ? U->data_ptr() : nullptr;
  {
    py::gil_scoped_release nogil;
    check(wc_conv_forward(&d, Input.data_ptr(), Weight.data_ptr(), s, up, bp, Output.data_ptr(), ws.data_ptr(), bytes, st));
  }
  return d.m;
}

std::vector<int> ints_of(py::object v, int nd, const char* what) {
  std::vector<int> r;
  if (py::isinstance<py::int_>(v)) {
    r.assign(nd, v.cast<int>());
  } else {
    r = v.cast<std::vector<int>>();
    if ((int)r.size() != nd) throw std::invalid_argument(std::string(what) + ": expected one int or " + std::to_string(nd) + " values");
  }
  return r;
}

// Winograd / DWM convolution of an NC[D]HW tensor with a (K, C, [kD,] kH, kW) filter; returns an NC[D]HW
// tensor whose memory is channel-last (or plain contiguous with channels_first_out).  A channel-last input is
// used without a copy and a contiguous channel-first one is handed to the library as it is
// (wc_conv_desc.x_layout); any other layout is made contiguous first.  The compiled form of the Python callers' common path (dwm.py:5-40, matrix_conv.py:70-135
// of the reference end in the same call).
at::Tensor conv_forward(at::Tensor x, at::Tensor w, std::optional<at::Tensor> bias, py::object stride, py::object padding,
                        int m, std::optional<at::Tensor> U, int chunk_images, bool whole_kernel, py::object stacked,
                        bool unfused, bool channels_first_out, py::object direct) {
  const int nd = (int)x.dim() - 2;
  if ((nd != 2 && nd != 3) || w.dim() != nd + 2)
    throw std::invalid_argument("expected 4-D or 5-D input and matching filter, got " + shape_str(x.sizes()) + " and " + shape_str(w.sizes()));
  if (x.size(1) != w.size(1))
    throw std::invalid_argument("input has " + std::to_string(x.size(1)) + " channels, filter expects " + std::to_string(w.size(1)) +
                                " (groups are not supported)");
  const int64_t K = w.size(0);
  if (bias && bias->defined()) {
    if (bias->dim() != 1 || bias->numel() != K)
      throw std::invalid_argument("bias must be a 1-D tensor of " + std::to_string(K) + " values (one per output channel), got shape " +
                                  shape_str(bias->sizes()));
    if (bias->scalar_type() != x.scalar_type()) {
      std::ostringstream os;
      os << "bias is " << bias->scalar_type() << ", the input is " << x.scalar_type() << ": they must share one dtype";
      throw py::type_error(os.str());
    }
    if (bias->device() != x.device()) throw std::invalid_argument("bias and input are on different devices");
  }
  if (U && U->defined()) {
    if (U->scalar_type() != x.scalar_type()) {
      std::ostringstream os;
      os << "the transformed filter is " << U->scalar_type() << ", the input is " << x.scalar_type()
         << ": transform the filter in the input's dtype";
      throw py::type_error(os.str());
    }
    if (U->device() != x.device()) throw std::invalid_argument("the transformed filter and the input are on different devices");
  }
  require_gpu(x, "conv_forward");
  require_gpu(w, "conv_forward");
  if (w.scalar_type() != x.scalar_type()) throw py::type_error("input, filter and bias must share one dtype");
  const auto st = ints_of(stride, nd, "stride");
  for (int a = 1; a < nd; ++a)
    if (st[a] != st[0]) { PyErr_SetString(PyExc_NotImplementedError, "stride must be the same on every axis"); throw py::error_already_set(); }
  const auto pd = ints_of(padding, nd, "padding");

  wc_conv_desc d{};
  d.ndim = nd;
  d.N = (int)(x.size(0) > 0 ? x.size(0) : 1);      // an empty batch: the shape arithmetic runs on one image
  d.C = (int)x.size(1); d.K = (int)K;
  d.in[0] = d.kernel[0] = 1;
  for (int a = 0; a < nd; ++a) {
    d.in[3 - nd + a] = (int)x.size(2 + a);
    d.kernel[3 - nd + a] = (int)w.size(2 + a);
    d.pad[3 - nd + a] = pd[a];
  }
  d.stride = st[0]; d.m = m; d.dtype = dtype_of(x);
  d.chunk_images = chunk_images;
  d.whole_kernel = whole_kernel;
  d.stacked = stacked.is_none() ? -1 : (py::isinstance<py::bool_>(stacked) ? (int)stacked.cast<bool>() : stacked.cast<int>());
  d.direct = direct.is_none() ? 0 : (direct.cast<bool>() ? 1 : -1);      // None: the library may choose it
  check(wc_conv_auto(&d));
  int out[3], grid[3];
  check(wc_conv_out_dims(&d, out, grid));
  std::vector<int64_t> ys{x.size(0)};                      // channel-last shape of y
  for (int a = 3 - nd; a < 3; ++a) ys.push_back(out[a]);
  ys.push_back(K);
  std::vector<int64_t> to_cl{0}, to_cf{0, nd + 1};
  for (int a = 0; a < nd; ++a) { to_cl.push_back(2 + a); to_cf.push_back(1 + a); }
  to_cl.push_back(1);
  std::vector<int64_t> ys_cf{ys[0], K};
  for (int a = 0; a < nd; ++a) ys_cf.push_back(ys[1 + a]);
  at::Tensor y = at::empty(channels_first_out ? ys_cf : ys, x.options());
  if (x.size(0) == 0) return channels_first_out ? y : y.permute(to_cf);
  at::Tensor x_mem = x.permute(to_cl);
  if (!x_mem.is_contiguous()) {                            // not channel-last memory: channel-first, read as it is
    x_mem = x.is_contiguous() ? x : x.contiguous();
    d.x_layout = 1;
  }
  d.y_layout = channels_first_out;
  auto misaligned = [](const at::Tensor& t) { return (reinterpret_cast<uintptr_t>(t.data_ptr()) & 15) != 0; };
  d.unfused = unfused || misaligned(x_mem) || (U && U->defined() && misaligned(*U));
  if (U && U->defined()) {
    size_t ue = 0;
    check(wc_conv_u_elems(&d, &ue));
    if (!U->is_contiguous() || (size_t)U->numel() != ue)
      throw std::invalid_argument("U has " + std::to_string(U->numel()) + " elements, this convolution needs a contiguous transformed "
                                  "filter of " + std::to_string(ue) + " (transform_filter must be called with the same options)");
  }
  size_t bytes = 0;
  check(wc_conv_workspace_bytes(&d, &bytes));
  void* stream = stream_of(x);
  at::Tensor ws = workspace_for(x, bytes, stream);
  at::Tensor bc = bias && bias->defined() ? bias->contiguous() : at::Tensor();
  int64_t s[5] = {w.stride(0), w.stride(1), 0, 0, 0};
  for (int a = 0; a < nd; ++a) s[5 - nd + a] = w.stride(2 + a);
  {
    py::gil_scoped_release nogil;
    check(wc_conv_forward(&d, x_mem.data_ptr(), w.data_ptr(), s, U && U->defined() ? U->data_ptr() : nullptr,
                          bc.defined() ? bc.data_ptr() : nullptr, y.data_ptr(), ws.data_ptr(), bytes, stream));
  }
  return channels_first_out ? y : y.permute(to_cf);
}

// The reference's native entry point (pybind/extern.hpp:7-9): VALID convolution.  The four scratch tensors
// of the reference signature (dwm.py:122-125) are accepted and ignored: the engine sizes its own workspace.
void DWM(at::Tensor Input, at::Tensor Weight, at::Tensor Output, int stride, py::object, py::object, py::object, py::object) {
  winograd_conv(Input, Weight, Output, std::nullopt, stride, py::int_(0), 2, "dwm", std::nullopt, 0, py::none());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.doc() = "MI355X-native stand-in for the reference extension MakePytorchBackend (pybind/bind.cpp:10-24)";
  static py::exception<WinoconvError> winoconv_error(m, "WinoconvError", PyExc_RuntimeError);
  py::register_exception_translator([](std::exception_ptr p) {
    try {
      if (p) std::rethrow_exception(p);
    } catch (const Unsupported& e) {
      PyErr_SetString(PyExc_NotImplementedError, e.what());
    }
  });
  py::class_<Foo>(m, "Foo")
      .def(py::init<>())
      .def("setKey", &Foo::setKey)
      .def("getKey", &Foo::getKey)
      .def("__repr__", [](const Foo& a) { return a.toString(); });
  m.def("AddGPU", &AddGPU);
  m.def("WinoSplit", &WinoSplit);
  m.def("WinoConcat", &WinoConcat);
  m.def("DWM", &DWM, py::arg("Input"), py::arg("Weight"), py::arg("Output"), py::arg("stride"),
        py::arg("tmp_input_buffer") = py::none(), py::arg("tmp_weight_buffer") = py::none(),
        py::arg("tmp_product_buffer") = py::none(), py::arg("tmp_ptr_buffer") = py::none());
  m.def("winograd_conv", &winograd_conv, py::arg("Input"), py::arg("Weight"), py::arg("Output"),
        py::arg("bias") = py::none(), py::arg("stride") = 1, py::arg("padding") = 0, py::arg("m") = 2,
        py::arg("algo") = "dwm", py::arg("U") = py::none(), py::arg("chunk_images") = 0, py::arg("stacked") = py::none());
  m.def("split_and_concat", &split_and_concat);
  m.def("conv_forward", &conv_forward, py::arg("x"), py::arg("w"), py::arg("bias") = py::none(), py::arg("stride") = 1,
        py::arg("padding") = 0, py::arg("m") = 2, py::arg("U") = py::none(), py::arg("chunk_images") = 0,
        py::arg("whole_kernel") = false, py::arg("stacked") = py::none(), py::arg("unfused") = false,
        py::arg("channels_first_out") = false, py::arg("direct") = py::none());
  m.def("version", []() { return std::string(wc_version()); });
}
