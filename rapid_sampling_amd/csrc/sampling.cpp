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
#include <c10/hip/HIPFunctions.h>

#include <map>
#include <mutex>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "rapid_sampling.h"

namespace {

// Way through the library that every call of this module asks for (RS_PATH_*): a hook for
// benchmarks and tests that compare the paths; results do not depend on it.
int g_forced_path = RS_PATH_AUTO;

void *current_stream(const at::Tensor &t)
{
    return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// One zero-initialised workspace per (device, stream), sized for the largest B
// and the largest V seen so far (the two maxima separately: that is what lets
// calls of different shapes share it), with the rs_policy object that routes
// the streaming path and carries asynchronous error reports.  The kernels
// leave the workspace clean, so it is never cleared again; calls that share
// it are ordered by the stream.  Takes the place of the reference's per-call
// `probs` scratch (sampling.cu:488,1014).
struct Entry {
    at::Tensor ws;
    int64_t B = 0, V = 0;
    rs_policy *policy = nullptr;
    bool captured = false;                  // a stream capture has recorded calls that point into ws
    std::vector<at::Tensor> retired;        // outgrown workspaces a captured graph may still point into
    std::vector<rs_policy *> retired_policies;   // replaced policies whose pinned words a captured graph's kernels may still write
};

bool is_capturing(void *stream)
{
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    return hipStreamIsCapturing((hipStream_t)stream, &cs) != hipSuccess || cs != hipStreamCaptureStatusNone;
}

// Entries live until the process ends (never destroyed: tensors must not be released after the
// runtime has shut down).  The last entry used by a thread is remembered, so that the steady state
// takes no lock and no map lookup.
Entry &entry_for(int device, void *stream)
{
    static std::mutex mu;
    static auto *cache = new std::map<std::pair<int, void *>, Entry *>();
    thread_local int last_device = -1;
    thread_local void *last_stream = nullptr;
    thread_local Entry *last = nullptr;
    if (last && last_device == device && last_stream == stream) return *last;
    std::lock_guard<std::mutex> lock(mu);
    Entry *&e = (*cache)[{device, stream}];
    if (!e) e = new Entry();
    last_device = device; last_stream = stream; last = e;
    return *e;
}

void init_workspace(Entry &e, void *stream)
{
    const int rc = rs_workspace_init(e.ws.data_ptr(), (size_t)e.ws.numel(), stream);
    if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
}

// Grows the entry's workspace to serve (B, V).  Under stream capture nothing may be allocated
// (the allocation would belong to the graph's private pool and the fill would be replayed with
// every launch of the graph): reserve_workspace(B, V) before capturing.
Entry &workspace_for(const at::Tensor &like, void *stream, int64_t B, int64_t V)
{
    Entry &e = entry_for((int)like.device().index(), stream);
    if (!e.ws.defined() || B > e.B || V > e.V) {
        if (is_capturing(stream))
            throw std::runtime_error("rapid_sampling: the workspace of this stream must grow for B=" + std::to_string(B) +
                                     ", V=" + std::to_string(V) + " while the stream is being captured; call "
                                     "reserve_workspace(B, V) on this stream before the capture begins");
        if (!e.policy && rs_policy_create(&e.policy) != RS_OK)
            throw std::runtime_error("rapid_sampling: could not allocate the pinned host words of the workspace");
        e.B = std::max(e.B, B);
        e.V = std::max(e.V, V);
        size_t bytes = 0;
        rs_workspace_bytes((int32_t)e.B, (int32_t)e.V, &bytes);
        if (e.ws.defined() && e.captured) e.retired.push_back(e.ws);      // otherwise nothing points into it any more
        e.captured = false;
        e.ws = at::empty({(int64_t)bytes}, at::TensorOptions().dtype(at::kChar).device(like.device()));
        init_workspace(e, stream);
    }
    return e;
}

// A kernel that gave up waiting for its peers (RS_ERR_DEVICE) leaves garbage in `out` and a dirty
// workspace.  It says so in a pinned host word, which is looked at -- without synchronising --
// before every call: the workspace is then set up again and the failure raised, one call late at
// the latest (workspace_status() synchronises and tells at once).
void raise_reported_failure(Entry &e, void *stream)
{
    int32_t err = RS_OK;
    if (!e.policy || rs_policy_error(e.policy, &err, 1) != RS_OK || err == RS_OK) return;
    if (!is_capturing(stream)) init_workspace(e, stream);
    throw std::runtime_error(std::string("rapid_sampling: an earlier sampling call on this stream failed (") +
                             rs_error_string(err) + "); its result was not valid. The workspace has been set up again.");
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
    Entry &e = workspace_for(logits, stream, s.B, s.V);
    raise_reported_failure(e, stream);
    if (!e.captured && is_capturing(stream)) e.captured = true;
    at::Tensor &ws = e.ws;
    rs_options opt;
    opt.path = g_forced_path; opt.slice_r = 0; opt.policy = e.policy;
    auto out = at::empty({s.B}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
    rs_row_diag *diag = nullptr;
    uint32_t *ebits = nullptr;
    if (dbg) {
        dbg->diag = at::zeros({s.B, (int64_t)sizeof(rs_row_diag)}, at::TensorOptions().dtype(at::kByte).device(logits.device()));
        dbg->e_bits = at::empty({s.B, s.V}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
        diag = (rs_row_diag *)dbg->diag.data_ptr();
        ebits = (uint32_t *)dbg->e_bits.data_ptr();
    }
    const int rc = rs_sample_ex(s.first_row, s.dtype, s.row_stride, penalties ? penalties->data_ptr<float>() : nullptr,
                                out.data_ptr<int32_t>(), inj ? nullptr : states->data_ptr(), inj,
                                (int32_t)s.B, (int32_t)s.V, (float)presence, (float)repetition, (float)decay,
                                c, k, p, ws.data_ptr(), (size_t)ws.numel(), diag, ebits, &opt, stream);
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

// Allocates and clears the workspace of the current stream of `device` for calls of up to B rows
// of up to V tokens.  Needed before a stream capture (nothing may be allocated while capturing);
// otherwise optional: the first call of a shape does the same.
void reserve_workspace(int64_t B, int64_t V, std::optional<int64_t> device)
{
    size_t bytes = 0;
    throw_for(rs_workspace_bytes((int32_t)B, (int32_t)V, &bytes), B, 1, V, 1.0);
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    workspace_for(like, current_stream(like), B, V);
}

// Synchronises the current stream of `device` and returns the sticky error word of its workspace:
// 0, or RS_ERR_DEVICE after a kernel gave up waiting (the workspace is then set up again, so the
// next call starts clean).
int64_t workspace_status(std::optional<int64_t> device)
{
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    void *stream = current_stream(like);
    Entry &e = entry_for((int)dev.index(), stream);
    if (!e.ws.defined()) return RS_OK;
    int32_t st = RS_OK;
    const int rc = rs_workspace_status(e.ws.data_ptr(), &st, stream);
    if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
    if (st != RS_OK) {
        int32_t dummy;
        if (e.policy) rs_policy_error(e.policy, &dummy, 1);
        init_workspace(e, stream);
    }
    return st;
}

// Routing state of the current stream's workspace (rs_policy_state): bit 0 set: calls without a
// bounding top_k currently take the general kernel (or a wide path), bit 1 set: calls with one take the
// general kernel, bit 2 set: calls that would take the one-pass wide path take the two-pass one, bit 3 set:
// calls that would take the two-pass wide path take the general kernel.  -1: no workspace yet.
int64_t policy_state(std::optional<int64_t> device)
{
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    Entry &e = entry_for((int)dev.index(), current_stream(like));
    int32_t st = -1;
    if (e.policy) rs_policy_state(e.policy, &st);
    return st;
}

// Forgets what the current stream's calls have learnt about routing: synchronises the stream, sets
// the workspace up again (so that the next streaming call does not report on the last one) and
// replaces the policy object.  For measurements that change workload on one stream and want each
// workload from a clean start; a service with one workload per stream never needs it.
void reset_routing(std::optional<int64_t> device)
{
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    void *stream = current_stream(like);
    if (is_capturing(stream)) throw std::runtime_error("rapid_sampling: reset_routing while the stream is being captured");
    Entry &e = entry_for((int)dev.index(), stream);
    if (!e.ws.defined()) return;
    if (hipStreamSynchronize((hipStream_t)stream) != hipSuccess) throw std::runtime_error("rapid_sampling: stream synchronisation failed");
    rs_policy *fresh = nullptr;
    if (rs_policy_create(&fresh) != RS_OK) throw std::runtime_error("rapid_sampling: could not allocate the pinned host words of the workspace");
    // A captured graph holds the address of the old policy's pinned words (its kernels report into them on
    // every replay): such a policy is kept, never freed, and simply no longer looked at.
    if (e.policy) {
        if (e.captured) e.retired_policies.push_back(e.policy);
        else rs_policy_destroy(e.policy);
    }
    e.policy = fresh;
    init_workspace(e, stream);
}

// Shortens (milliseconds > 0) or restores (0) the bound of the kernels' waits on the current
// stream's workspace.  For tests of the error path.
void set_wait_limit(int64_t milliseconds, std::optional<int64_t> device)
{
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    void *stream = current_stream(like);
    Entry &e = entry_for((int)dev.index(), stream);
    if (!e.ws.defined()) throw std::runtime_error("rapid_sampling: no workspace on this stream yet");
    const int rc = rs_workspace_set_wait_limit(e.ws.data_ptr(), (uint32_t)milliseconds, stream);
    if (rc != RS_OK) throw std::runtime_error(std::string("rapid_sampling: ") + rs_error_string(rc));
}

void force_path(const std::string &name)
{
    if (name == "auto") g_forced_path = RS_PATH_AUTO;
    else if (name == "cluster") g_forced_path = RS_PATH_CLUSTER;
    else if (name == "stream") g_forced_path = RS_PATH_STREAM;
    else if (name == "attempt") g_forced_path = RS_PATH_ATTEMPT;
    else if (name == "fused") g_forced_path = RS_PATH_FUSED;
    else if (name == "wide") g_forced_path = RS_PATH_WIDE;
    else if (name == "wide1") g_forced_path = RS_PATH_WIDE1;
    else if (name == "row") g_forced_path = RS_PATH_ROW;
    else throw std::invalid_argument("force_path: auto | cluster | stream | attempt | fused | wide | wide1 | row");
}

// The workspace tensor of the current stream (tests poison it to force the error path).
at::Tensor debug_workspace(std::optional<int64_t> device)
{
    const auto dev = at::Device(at::kCUDA, (c10::DeviceIndex)(device ? *device : c10::hip::current_device()));
    auto like = at::empty({1}, at::TensorOptions().dtype(at::kChar).device(dev));
    Entry &e = entry_for((int)dev.index(), current_stream(like));
    if (!e.ws.defined()) throw std::runtime_error("rapid_sampling: no workspace on this stream yet");
    return e.ws;
}

// Launch-plus-one-read floor kernel on the logits' grid (measurement aid).
at::Tensor floor_read(at::Tensor &logits, int64_t variant)
{
    const Shape s = read_logits(logits, std::nullopt, false);
    c10::hip::HIPGuardMasqueradingAsCUDA guard(logits.device());
    // not cleared: the kernel max-combines into it, and a second launch to zero it would be timed along
    auto out = at::empty({s.B}, at::TensorOptions().dtype(at::kInt).device(logits.device()));
    const int rc = rs_floor_read(static_cast<const float *>(s.first_row), s.row_stride, out.data_ptr<int32_t>(), (int32_t)s.B, (int32_t)s.V,
                                 (int32_t)variant, current_stream(logits));
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
    m.def("floor_read", &floor_read, py::arg("logits"), py::arg("variant") = 1);
    m.def("reserve_workspace", &reserve_workspace, py::arg("B"), py::arg("V"), py::arg("device") = py::none());
    m.def("workspace_status", &workspace_status, py::arg("device") = py::none());
    m.def("policy_state", &policy_state, py::arg("device") = py::none());
    m.def("force_path", &force_path, py::arg("name"));
    m.def("reset_routing", &reset_routing, py::arg("device") = py::none());
    m.def("debug_workspace", &debug_workspace, py::arg("device") = py::none());
    m.def("set_wait_limit", &set_wait_limit, py::arg("milliseconds"), py::arg("device") = py::none());
    m.attr("STATE_BYTES_PER_ROW") = RS_STATE_BYTES_PER_ROW;
    m.attr("DIAG_BYTES") = (int)sizeof(rs_row_diag);
}
