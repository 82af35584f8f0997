// Host side of the sampler: the PyTorch-ROCm extension module.
//
// Mirrors the reference's three entry points (/root/reference/sampling.cpp:2-8;
// wrappers at /root/reference/sampling.cu:140-144, :440-515, :968-1044): same
// names, same positional argument order, same shapes and limits, the same
// std::invalid_argument (Python ValueError) for the same conditions.  Tensors
// stay torch's; everything below the tensor layer goes through the C ABI of
// include/rapid_sampling.h.  PyTorch supplies device memory and the current
// stream, nothing else.
#include <torch/extension.h>
#include <hip/hip_runtime_api.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <map>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "rapid_sampling.h"

namespace {

void *current_stream(const at::Tensor &t)
{
    return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// One zero-initialised workspace per (device, stream), sized for the largest B
// and the largest V seen so far (the two maxima separately: that is what lets
// calls of different shapes share it).  The kernels leave it clean, so it is
// never cleared again; calls that share it are ordered by the stream.  Takes
// the place of the reference's per-call `probs` scratch (sampling.cu:488,1014).
at::Tensor &workspace_for(const at::Tensor &like, void *stream, int64_t B, int64_t V)
{
    // `retired` keeps outgrown workspaces alive: a captured HIP graph may still point into one
    struct Entry { at::Tensor ws; int64_t B = 0, V = 0; std::vector<at::Tensor> retired; };
    static std::mutex mu;
    static std::map<std::pair<int, void *>, Entry> cache;
    std::lock_guard<std::mutex> lock(mu);
    Entry &e = cache[{(int)like.device().index(), stream}];
    if (!e.ws.defined() || B > e.B || V > e.V) {
        e.B = std::max(e.B, B);
        e.V = std::max(e.V, V);
        size_t bytes = 0;
        rs_workspace_bytes((int32_t)e.B, (int32_t)e.V, &bytes);
        if (e.ws.defined()) e.retired.push_back(e.ws);
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        const bool capturing = hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone;
        if (capturing) {
            // a memset must not be recorded into a graph: clear with a fill kernel, and do without
            // the routing reports rs_workspace_init would set up
            e.ws = at::zeros({(int64_t)bytes}, at::TensorOptions().dtype(at::kChar).device(like.device()));
        } else {
            e.ws = at::empty({(int64_t)bytes}, at::TensorOptions().dtype(at::kChar).device(like.device()));
            const int rc = rs_workspace_init(e.ws.data_ptr(), bytes, stream);
            if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
        }
    }
    return e.ws;
}

void throw_for(int code, int64_t B, int64_t T, int64_t V, double temperature)
{
    switch (code) {
    case RS_OK:
        return;
    case RS_ERR_VOCAB:
        throw std::invalid_argument("Vocabulary size must be multiple of 4, and no larger than 1048576, got " +
                                    std::to_string(V) + " !\n");
    case RS_ERR_BATCH:
        throw std::invalid_argument("B and T must be positive, got B=" + std::to_string(B) + ", T=" +
                                    std::to_string(T) + " !\n");
    case RS_ERR_TEMPERATURE:
        throw std::invalid_argument("Temperature outside range, got " + std::to_string(temperature) +
                                    ", expect [0.001, 1000]!\n");
    default:
        throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(code));
    }
}

struct Shape {
    int64_t B, T, V;
    const void *first_row;    // logits[:, T-1, :] start
    int64_t row_stride;
    int32_t dtype;            // RS_DTYPE_*
};

// Shapes as the reference reads them (sampling.cu:458-460, :982-984), plus the
// checks it omits: device, unit stride of the vocabulary axis.
// The reference takes float32 logits only (sampling.cu:452-457, :976-981), and so does this unless
// the caller passes accept_half=True: then bfloat16 and float16 logits are read as they are (they
// widen to float32 exactly; half the bytes).
int32_t logits_dtype(const at::Tensor &logits, bool accept_half)
{
    if (logits.dtype() == at::kFloat) return RS_DTYPE_F32;
    if (accept_half && logits.dtype() == at::kBFloat16) return RS_DTYPE_BF16;
    if (accept_half && logits.dtype() == at::kHalf) return RS_DTYPE_F16;
    throw std::invalid_argument("Logits tensor must be of type float32 (FP32), got " +
                                std::string(logits.dtype().name()) + " !\n");
}

Shape read_logits(const at::Tensor &logits, std::optional<int64_t> B_override, bool accept_half)
{
    const int32_t dtype = logits_dtype(logits, accept_half);
    if (logits.dim() < 1 || logits.dim() > 3)
        throw std::invalid_argument("Logits tensor must have shape (V,), (B, V) or (B, T, V) !\n");
    Shape s;
    s.V = logits.size(-1);
    s.B = B_override ? *B_override : (logits.dim() >= 2 ? logits.size(0) : 1);
    s.T = logits.dim() == 3 ? logits.size(1) : 1;
    if (!(s.V > 0 && s.V <= 1048576 && s.V % 4 == 0)) throw_for(RS_ERR_VOCAB, s.B, s.T, s.V, 0);
    if (!(s.B > 0 && s.T > 0)) throw_for(RS_ERR_BATCH, s.B, s.T, s.V, 0);
    const int64_t rows = logits.dim() >= 2 ? logits.size(0) : 1;
    if (s.B > rows) throw std::invalid_argument("penalties has more rows than logits !\n");
    s.row_stride = logits.dim() >= 2 ? logits.stride(0) : s.V;
    const int64_t t_stride = logits.dim() == 3 ? logits.stride(1) : 0;
    s.first_row = static_cast<const char *>(logits.data_ptr()) + (s.T - 1) * t_stride * (int64_t)logits.element_size();
    s.dtype = dtype;
    return s;
}

void check_states(const at::Tensor &states, const at::Tensor &logits, int64_t B)
{
    if (!states.is_cuda() || states.device() != logits.device() || !states.is_contiguous() ||
        (int64_t)states.nbytes() < B * RS_STATE_BYTES_PER_ROW)
        throw std::invalid_argument("states must be the tensor returned by setup_rand(seed, B) for at least B=" +
                                    std::to_string(B) + " rows, on the logits' device !\n");
}

const float *check_uniforms(const std::optional<at::Tensor> &u, const at::Tensor &logits, int64_t B)
{
    if (!u) return nullptr;
    if (u->dtype() != at::kFloat || !u->is_cuda() || u->device() != logits.device() || !u->is_contiguous() ||
        u->numel() != B)
        throw std::invalid_argument("uniforms must be a contiguous float32 GPU tensor of B elements !\n");
    return u->data_ptr<float>();
}

void check_penalties(const at::Tensor &penalties, const at::Tensor &logits, const Shape &s)
{
    if (penalties.dtype() != at::kFloat || !penalties.is_cuda() || penalties.device() != logits.device() ||
        !penalties.is_contiguous() || penalties.size(-1) != s.V || penalties.dim() < 1 || penalties.dim() > 2)
        throw std::invalid_argument("penalties must be a contiguous float32 GPU tensor of shape (B, V) !\n");
}

struct Debug {
    at::Tensor diag;     // (B, sizeof(rs_row_diag)) uint8
    at::Tensor e_bits;   // (B, V) int32
};

at::Tensor run(const at::Tensor &logits, const Shape &s, at::Tensor *penalties, const at::Tensor *states,
               double presence, double repetition, double decay, double temperature, int64_t top_k, double top_p,
               const std::optional<at::Tensor> &uniforms, Debug *dbg)
{
    float c, p;
    int32_t k;
    throw_for(rs_normalize_args(temperature, top_k, top_p, s.B, s.T, s.V, &c, &k, &p), s.B, s.T, s.V, temperature);
    // checks the reference leaves out, after the ones it makes
    if (!logits.is_cuda()) throw std::invalid_argument("Logits tensor must live on the GPU !\n");
    if (logits.stride(-1) != 1) throw std::invalid_argument("Logits tensor must be contiguous along the vocabulary axis !\n");
    if (penalties) check_penalties(*penalties, logits, s);
    const float *inj = check_uniforms(uniforms, logits, s.B);
    if (!inj) check_states(*states, logits, s.B);

    c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
    void *stream = current_stream(logits);
    size_t bytes = 0;
    throw_for(rs_workspace_bytes((int32_t)s.B, (int32_t)s.V, &bytes), s.B, s.T, s.V, temperature);
    at::Tensor &ws = workspace_for(logits, stream, s.B, s.V);
    auto out = at::empty({s.B}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
    rs_row_diag *diag = nullptr;
    uint32_t *ebits = nullptr;
    if (dbg) {
        dbg->diag = at::zeros({s.B, (int64_t)sizeof(rs_row_diag)}, at::TensorOptions().dtype(at::kByte).device(logits.device()));
        dbg->e_bits = at::empty({s.B, s.V}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
        diag = (rs_row_diag *)dbg->diag.data_ptr();
        ebits = (uint32_t *)dbg->e_bits.data_ptr();
    }
    const int rc = rs_sample_dtype(s.first_row, s.dtype, s.row_stride, penalties ? penalties->data_ptr<float>() : nullptr,
                                   out.data_ptr<int32_t>(), inj ? nullptr : states->data_ptr(), inj,
                                   (int32_t)s.B, (int32_t)s.V, (float)presence, (float)repetition, (float)decay,
                                   c, k, p, ws.data_ptr(), (size_t)ws.numel(), diag, ebits, stream);
    throw_for(rc, s.B, s.T, s.V, temperature);
    return out;
}

}  // namespace

// sampling.cu:140-144.  State is 64 bytes per row, opaque to the caller.
at::Tensor setup_rand(int64_t seed, int64_t B)
{
    if (B <= 0) throw std::invalid_argument("B must be positive, got B=" + std::to_string(B) + " !\n");
    auto state = at::zeros({B * RS_STATE_BYTES_PER_ROW}, at::TensorOptions().dtype(at::kChar).device(at::kCUDA));
    const int rc = rs_philox_init(state.data_ptr(), (uint64_t)seed, (int32_t)B, current_stream(state));
    if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
    return state;
}

// sampling.cu:968-1044
at::Tensor batch_sampling_temperature_topk_topp(at::Tensor &logits, at::Tensor &states, double temperature,
                                                int64_t top_k, double top_p, std::optional<at::Tensor> uniforms,
                                                bool accept_half)
{
    const Shape s = read_logits(logits, std::nullopt, accept_half);
    return run(logits, s, nullptr, &states, 0, 0, 1, temperature, top_k, top_p, uniforms, nullptr);
}

// sampling.cu:440-515.  B comes from penalties, as in the reference (:459).
at::Tensor batch_sampling_repetition_temperature_topk_topp(at::Tensor &logits, at::Tensor &penalties,
                                                           at::Tensor &states, double presence_penalty,
                                                           double repetition_penalty, double penalty_decay,
                                                           double temperature, int64_t top_k, double top_p,
                                                           std::optional<at::Tensor> uniforms, bool accept_half)
{
    logits_dtype(logits, accept_half);                   // the reference's first check (sampling.cu:452)
    const int64_t B = penalties.dim() == 2 ? penalties.size(0) : 1;
    const Shape s = read_logits(logits, B, accept_half);
    return run(logits, s, &penalties, &states, presence_penalty, repetition_penalty, penalty_decay, temperature,
               top_k, top_p, uniforms, nullptr);
}

// Same call with the per-row diagnostics and the e bit patterns returned too
// (tests compare them with the CPU oracle).  penalties may be None.
std::tuple<at::Tensor, at::Tensor, at::Tensor> batch_sampling_debug(
    at::Tensor &logits, std::optional<at::Tensor> penalties, std::optional<at::Tensor> states,
    double presence_penalty, double repetition_penalty, double penalty_decay, double temperature, int64_t top_k,
    double top_p, std::optional<at::Tensor> uniforms, bool accept_half)
{
    std::optional<int64_t> B;
    if (penalties) B = penalties->dim() == 2 ? penalties->size(0) : 1;
    const Shape s = read_logits(logits, B, accept_half);
    if (!uniforms && !states) throw std::invalid_argument("need states or uniforms !\n");
    Debug dbg;
    at::Tensor out = run(logits, s, penalties ? &*penalties : nullptr, states ? &*states : nullptr, presence_penalty,
                         repetition_penalty, penalty_decay, temperature, top_k, top_p, uniforms, &dbg);
    return {out, dbg.diag, dbg.e_bits};
}

// Launch-plus-one-read floor kernel on the logits' grid (measurement aid).
at::Tensor floor_read(at::Tensor &logits)
{
    const Shape s = read_logits(logits, std::nullopt, false);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
    // not cleared: the kernel max-combines into it, and a second launch to zero it would be timed along
    auto out = at::empty({s.B}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
    const int rc = rs_floor_read(static_cast<const float *>(s.first_row), s.row_stride, out.data_ptr<int32_t>(), (int32_t)s.B, (int32_t)s.V,
                                 current_stream(logits));
    if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
    return out;
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    namespace py = pybind11;
    m.def("setup_rand", &setup_rand, py::arg("seed"), py::arg("B"));
    m.def("batch_sampling_repetition_temperature_topk_topp", &batch_sampling_repetition_temperature_topk_topp,
          py::arg("logits"), py::arg("penalties"), py::arg("states"), py::arg("presence_penalty"),
          py::arg("repetition_penalty"), py::arg("penalty_decay"), py::arg("temperature"), py::arg("top_k"),
          py::arg("top_p"), py::kw_only(), py::arg("uniforms") = py::none(), py::arg("accept_half") = false);
    m.def("batch_sampling_temperature_topk_topp", &batch_sampling_temperature_topk_topp, py::arg("logits"),
          py::arg("states"), py::arg("temperature"), py::arg("top_k"), py::arg("top_p"), py::kw_only(),
          py::arg("uniforms") = py::none(), py::arg("accept_half") = false);
    m.def("batch_sampling_debug", &batch_sampling_debug, py::arg("logits"), py::arg("penalties"), py::arg("states"),
          py::arg("presence_penalty"), py::arg("repetition_penalty"), py::arg("penalty_decay"),
          py::arg("temperature"), py::arg("top_k"), py::arg("top_p"), py::kw_only(),
          py::arg("uniforms") = py::none(), py::arg("accept_half") = false);
    m.def("floor_read", &floor_read, py::arg("logits"));
    m.attr("STATE_BYTES_PER_ROW") = RS_STATE_BYTES_PER_ROW;
    m.attr("DIAG_BYTES") = (int)sizeof(rs_row_diag);
}
