// Torch C++ extension with the reference's pybind surface for the codec pipeline
// (custom/custom_kernel.cpp:194-321): the AbstractCompressor classes, their registry, and
// compress_operation / comm_operation / decompress_operation / clear_ptr_lst, plus
// torch.ops.tutel_ops.cumsum (custom_kernel.cpp:331-385).  All device work goes through the C
// ABI of libplanmoe_hip; this file only owns tensors and object lifetimes.
// One GPU: the comm step is a device copy into g_output, issued on a comm stream of its own (same
// priority as the compute stream) under the reference's event protocol, so that with
// a2a_ffn_overlap_degree > 1 a chunk's copy runs beside the next chunk's compress.
#include "planmoe/compressor/abstract.h"
#include "planmoe/compressor/int8.h"
#include "planmoe/compressor/lz.h"
#include "planmoe/compressor/no.h"
#include "planmoe/compressor/zfpc.h"
#include "planmoe/compressor/registry.h"
#include "planmoe_hip.h"

#include <ATen/hip/HIPEvent.h>
#include <hip/hip_runtime_api.h>
#include <map>
#include <torch/script.h>

static void *current_stream() { return (void *)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream(); }

static int pm_dtype(const torch::Tensor &t)
{
    switch (t.scalar_type()) {
    case at::kFloat: return PLANMOE_F32;
    case at::kBFloat16: return PLANMOE_BF16;
    case at::kHalf: return PLANMOE_F16;
    default: AT_ASSERTM(false, "planmoe: unsupported dtype (float32, bfloat16 or float16)"); return -1;
    }
}
#define PM_CALL(expr) AT_ASSERTM((expr) == 0, planmoe_last_error())
#define CHECK_GPU(x) AT_ASSERTM((x).is_cuda(), #x " must be a GPU tensor (this build has no CPU path)")

// ---------------------------------------------------------------- comm
AbstractComm::AbstractComm(std::vector<PlanMoEStream> *stream, std::vector<ncclComm_t> g_nccl_comm,
                           const int &g_world_size, const int &g_world_rank, const int &g_local_size,
                           const int &g_local_rank) :
    stream(stream), g_nccl_comm(g_nccl_comm), g_world_size(g_world_size), g_world_rank(g_world_rank),
    g_local_size(g_local_size), g_local_rank(g_local_rank) {}
void AbstractComm::pre_comm(const torch::Tensor &) {}
AbstractComm::~AbstractComm() {}

IdentityComm::IdentityComm(std::vector<PlanMoEStream> *stream, std::vector<ncclComm_t> comm, const int &ws,
                           const int &wr, const int &ls, const int &lr) :
    AbstractComm(stream, comm, ws, wr, ls, lr) {}
void IdentityComm::all_to_all(const torch::Tensor &input, const torch::Tensor &output, size_t length)
{
    AT_ASSERTM(g_world_size == 1, "IdentityComm is the one-GPU all-to-all");
    // on the comm stream (naive.cpp:11-27 issues its send / recv pairs on stream->at(0)); the caller
    // has made that stream wait for the producer of `input`
    hipStream_t st = (stream && !stream->empty()) ? (hipStream_t)stream->at(0).stream() : (hipStream_t)current_stream();
    AT_ASSERTM(hipMemcpyAsync(output.data_ptr(), input.data_ptr(), length, hipMemcpyDeviceToDevice, st) == hipSuccess,
               "all_to_all copy failed");
}

// ---------------------------------------------------------------- compressors
AbstractCompressor::AbstractCompressor(std::shared_ptr<AbstractComm> comm_ptr) { this->comm_ptr = comm_ptr; }
AbstractCompressor::~AbstractCompressor() { comm_ptr.reset(); }
void AbstractCompressor::pre_comm(const PlanMoEStream *) {}

NoCompressor::NoCompressor(std::shared_ptr<AbstractComm> comm_ptr) : AbstractCompressor(comm_ptr) {}
torch::Tensor NoCompressor::compress(const torch::Tensor &input)
{
    g_output = at::empty_like(input);
    return input;
}
torch::Tensor NoCompressor::decompress(const torch::Tensor &input) { return input; }
void NoCompressor::all_to_all(const torch::Tensor &input, const torch::Tensor &output)
{
    comm_ptr->all_to_all(input, output, input.nbytes());
}

Int8Compressor::Int8Compressor(std::shared_ptr<AbstractComm> comm_ptr) : AbstractCompressor(comm_ptr) {}
torch::Tensor Int8Compressor::compress(const torch::Tensor &input_)
{
    CHECK_GPU(input_);
    const torch::Tensor input = input_.contiguous();
    sizes = input.sizes().vec();
    dtype = input.dtype();
    length = (size_t)input.numel();
    AT_ASSERTM(!sizes.empty() && sizes.back() > 0, "int8: empty rows");
    const int64_t M = sizes.back(), rows = input.numel() / M;
    std::vector<int64_t> rshape(sizes.begin(), sizes.end());
    rshape.back() = 1;
    bias = torch::empty(rshape, input.options());
    scale = torch::empty(rshape, input.options());
    torch::Tensor fp_output = torch::empty({(int64_t)((length + 3) / 4)}, input.options().dtype(at::kFloat));
    PM_CALL(planmoe_int8_compress(input.data_ptr(), pm_dtype(input), rows, (int)M, (uint8_t *)fp_output.data_ptr(),
                                  bias.data_ptr(), scale.data_ptr(), current_stream()));
    g_bias = at::empty_like(bias);
    g_scale = at::empty_like(scale);
    this->g_output = at::empty_like(fp_output);
    // the comm stream reads bias / scale and writes their receive-side twins (int8.cpp:25-42)
    for (auto &comm_stream : *comm_ptr->stream)
        for (const torch::Tensor *t : {&bias, &scale, &g_bias, &g_scale, &g_output}) t->record_stream(comm_stream);
    return fp_output;
}
torch::Tensor Int8Compressor::decompress(const torch::Tensor &input)
{
    CHECK_GPU(input);
    std::vector<int64_t> shape(sizes.begin(), sizes.end());
    torch::Tensor output = torch::empty(shape, input.options().dtype(dtype));
    const int64_t M = sizes.back(), rows = output.numel() / M;
    PM_CALL(planmoe_int8_decompress((const uint8_t *)input.data_ptr(), g_bias.data_ptr(), g_scale.data_ptr(),
                                    pm_dtype(output), rows, (int)M, output.data_ptr(), current_stream()));
    return output;
}
void Int8Compressor::pre_comm(const PlanMoEStream *) {}
void Int8Compressor::all_to_all(const torch::Tensor &input, const torch::Tensor &output)
{
    comm_ptr->all_to_all(input, output, length);
    comm_ptr->all_to_all(bias, g_bias, bias.nbytes());
    comm_ptr->all_to_all(scale, g_scale, scale.nbytes());
}

ZfpCompressor::ZfpCompressor(std::shared_ptr<AbstractComm> comm_ptr, double compress_rate) noexcept :
    AbstractCompressor(comm_ptr)
{
    this->compress_rate = compress_rate;
    this->buffer = nullptr;
    this->last_bufsize = 0;
}
ZfpCompressor::~ZfpCompressor() { buffer = nullptr; }
// zfpc.h:15 -- the reference hands zfp's CUDA back end a stream; here every launch goes to the
// current stream, the value is only kept
void ZfpCompressor::set_cuda_stream(const hipStream_t &s) { this->cuda_stream = s; }
void ZfpCompressor::set_compress_rate(const double &rate) { this->compress_rate = rate; }
torch::Tensor ZfpCompressor::compress(const torch::Tensor &input_)
{
    CHECK_GPU(input_);
    const torch::Tensor input = input_.contiguous();
    sizes = input.sizes().vec();
    AT_ASSERTM(sizes.size() == 3, "zfp fails.");
    AT_ASSERTM(sizes[0] % 4 == 0, "zfp fails.");
    AT_ASSERTM(sizes[1] % 4 == 0, "zfp fails.");
    AT_ASSERTM(sizes[2] % 4 == 0, "zfp fails.");
    AT_ASSERTM(input.scalar_type() == at::kFloat, "zfp: the codec reads the buffer as fp32; pass a float32 tensor");
    const int64_t nx = sizes[2], ny = sizes[1] * sizes[0];
    const size_t bufsize = planmoe_zfp_max_bytes(2, nx, ny, compress_rate);
    torch::Tensor output = torch::zeros({(int64_t)((bufsize + 1) / 2)}, input.options().dtype(at::kHalf));
    PM_CALL(planmoe_zfp_compress((const float *)input.data_ptr(), 2, nx, ny, compress_rate, output.data_ptr(),
                                 bufsize, current_stream()));
    length = planmoe_zfp_stream_bytes(2, nx, ny, compress_rate);
    g_output = torch::empty_like(output);
    return output;
}
torch::Tensor ZfpCompressor::decompress(const torch::Tensor &input)
{
    CHECK_GPU(input);
    std::vector<int64_t> shape(sizes.begin(), sizes.end());
    torch::Tensor output = torch::empty(shape, input.options().dtype(at::kFloat));
    PM_CALL(planmoe_zfp_decompress(input.data_ptr(), 2, sizes[2], sizes[1] * sizes[0], compress_rate,
                                   (float *)output.data_ptr(), current_stream()));
    return output;
}
void ZfpCompressor::all_to_all(const torch::Tensor &input, const torch::Tensor &output)
{
    comm_ptr->all_to_all(input, output, length);
}

LzCompressor::LzCompressor(std::shared_ptr<AbstractComm> comm_ptr) : AbstractCompressor(comm_ptr) {}
torch::Tensor LzCompressor::compress(const torch::Tensor &input)
{
    CHECK_GPU(input);
    AT_ASSERTM(input.scalar_type() == at::kFloat, "lz: expected scalar type Float");
    AT_ASSERTM(comm_ptr->g_world_size == 1, "lz: one slice per rank, and this build runs one rank");
    const torch::Tensor x = input.contiguous();
    const int64_t nbytes = (int64_t)x.nbytes();
    const int64_t blocks = planmoe_lz_blocks(nbytes);
    const auto i32 = x.options().dtype(at::kInt), u8 = x.options().dtype(at::kByte);
    flagArrOffsetGlobal        = at::empty({blocks + 1}, i32);
    compressedDataOffsetGlobal = at::empty({blocks + 1}, i32);
    flagArrGlobal              = at::empty({blocks * 64}, u8);          // the codec zeroes the slack itself
    compressedDataGlobal       = at::empty({blocks * 2048}, u8);
    workspace                  = at::empty({(int64_t)planmoe_lz_workspace_bytes(nbytes)}, u8);
    PM_CALL(planmoe_lz_compress(x.data_ptr(), nbytes, flagArrOffsetGlobal.data_ptr<int>(),
                                compressedDataOffsetGlobal.data_ptr<int>(), flagArrGlobal.data_ptr<uint8_t>(),
                                compressedDataGlobal.data_ptr<uint8_t>(), workspace.data_ptr(),
                                (size_t)workspace.nbytes(), current_stream()));
    g_flagArrOffsetGlobal        = at::empty_like(flagArrOffsetGlobal);
    g_compressedDataOffsetGlobal = at::empty_like(compressedDataOffsetGlobal);
    g_flagArrGlobal              = at::empty_like(flagArrGlobal);
    g_compressedDataGlobal       = at::empty_like(compressedDataGlobal);
    g_output                     = at::zeros_like(x);
    return input;
}
torch::Tensor LzCompressor::decompress(const torch::Tensor &input)
{
    CHECK_GPU(input);
    AT_ASSERTM(input.is_contiguous() && input.scalar_type() == at::kFloat, "lz: expected a contiguous Float tensor");
    PM_CALL(planmoe_lz_decompress(input.data_ptr(), (int64_t)input.nbytes(), g_flagArrOffsetGlobal.data_ptr<int>(),
                                  g_compressedDataOffsetGlobal.data_ptr<int>(), g_flagArrGlobal.data_ptr<uint8_t>(),
                                  g_compressedDataGlobal.data_ptr<uint8_t>(), current_stream()));
    return input;
}
void LzCompressor::all_to_all(const torch::Tensor &, const torch::Tensor &)
{
    // lz.cpp:67-73: the four stream tensors travel whole; input / output are not touched
    comm_ptr->all_to_all(flagArrOffsetGlobal, g_flagArrOffsetGlobal, flagArrOffsetGlobal.nbytes());
    comm_ptr->all_to_all(compressedDataOffsetGlobal, g_compressedDataOffsetGlobal, compressedDataOffsetGlobal.nbytes());
    comm_ptr->all_to_all(flagArrGlobal, g_flagArrGlobal, flagArrGlobal.nbytes());
    comm_ptr->all_to_all(compressedDataGlobal, g_compressedDataGlobal, compressedDataGlobal.nbytes());
}

// ---------------------------------------------------------------- registry (custom_kernel.cpp:194-288)
// one comm stream per device, taken from torch's pool at default priority the first time it is
// needed (the reference's g_nccl_stream, custom_kernel.cpp:128-153), and one event per
// compress / comm / decompress triple (g_cuda_events)
static std::map<int, std::vector<PlanMoEStream>> g_streams_by_device;
static std::vector<at::cuda::CUDAEvent> g_events;

static std::vector<PlanMoEStream> *comm_streams()
{
    const int dev = (int)c10::hip::current_device();
    auto it = g_streams_by_device.find(dev);
    if (it == g_streams_by_device.end())
        it = g_streams_by_device.emplace(dev, std::vector<PlanMoEStream>{
                 c10::hip::getStreamFromPoolMasqueradingAsCUDA(/*isHighPriority=*/false)}).first;
    return &it->second;
}

static std::map<std::string, planmoe::CompressorFactory> &factories()
{
    static std::map<std::string, planmoe::CompressorFactory> f;
    return f;
}
void planmoe::register_compressor(const std::string &name, planmoe::CompressorFactory factory) { factories()[name] = factory; }
std::vector<std::string> planmoe::registered_compressors()
{
    std::vector<std::string> names;
    for (auto &kv : factories()) names.push_back(kv.first);
    return names;
}

static AbstractCompressor *get_compressor(const std::string &name, std::shared_ptr<AbstractComm> comm_ptr)
{
    auto it = factories().find(name);                       // plug-ins first: they may replace a built-in name
    if (it != factories().end()) return it->second(comm_ptr);
    if (name == "int8") return new Int8Compressor(comm_ptr);
    if (name == "zfp") return new ZfpCompressor(comm_ptr);
    if (name == "lz") return new LzCompressor(comm_ptr);
    return new NoCompressor(comm_ptr);
}
static std::shared_ptr<AbstractComm> get_comm(const std::string &)
{
    // naive / pipe / dd / hetu are all the identity on one GPU
    return std::make_shared<IdentityComm>(comm_streams(), std::vector<ncclComm_t>(), 1, 0, 1, 0);
}

static std::vector<AbstractCompressor *> compress_ptr_lst;
static int comm_cnt = 0;
static int decompress_cnt = 0;

static void clear_ptr_lst()
{
    for (auto &p : compress_ptr_lst) { delete p; p = nullptr; }
    compress_ptr_lst.resize(0);
    comm_cnt = 0;
    decompress_cnt = 0;
}
// custom_kernel.cpp:242-258: the event of slot idx is recorded behind the compress on the compute stream
static torch::Tensor compress_operation(const torch::Tensor &input, const std::string &str, const std::string &comm_name)
{
    CHECK_GPU(input);                      // before anything asks the device for a stream
    const size_t idx = compress_ptr_lst.size();
    compress_ptr_lst.emplace_back(get_compressor(str, get_comm(comm_name)));
    torch::Tensor after_compress = compress_ptr_lst.back()->compress(input);
    if (g_events.size() <= idx) g_events.resize(idx + 1);
    g_events[idx].record(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
    for (auto &comm_stream : *comm_streams()) after_compress.record_stream(comm_stream);
    return after_compress;
}
// custom_kernel.cpp:260-277: the comm stream waits for the compress, carries the all-to-all, and
// records the event again
static torch::Tensor comm_operation(const torch::Tensor &input)
{
    AT_ASSERTM(comm_cnt < (int)compress_ptr_lst.size() && compress_ptr_lst[comm_cnt],
               "comm_operation: no matching compress_operation");
    const int idx = comm_cnt++;
    const PlanMoEStream original_stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA();
    compress_ptr_lst[idx]->pre_comm(&original_stream);
    for (auto &comm_stream : *comm_streams()) g_events[idx].block(comm_stream);
    compress_ptr_lst[idx]->all_to_all(input, compress_ptr_lst[idx]->g_output);
    for (auto &comm_stream : *comm_streams()) {
        g_events[idx].record(comm_stream);
        compress_ptr_lst[idx]->g_output.record_stream(comm_stream);
    }
    return compress_ptr_lst[idx]->g_output;
}
// custom_kernel.cpp:279-288: the compute stream waits for the all-to-all
static torch::Tensor decompress_operation(const torch::Tensor &input)
{
    AT_ASSERTM(decompress_cnt < (int)compress_ptr_lst.size() && compress_ptr_lst[decompress_cnt],
               "decompress_operation: no matching compress_operation");
    const int idx = decompress_cnt++;
    g_events[idx].block(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA());
    torch::Tensor output = compress_ptr_lst[idx]->decompress(input);
    delete compress_ptr_lst[idx];
    compress_ptr_lst[idx] = nullptr;
    return output;
}

// ---- invoke_cpu_fp32 / invoke_cpu_fp64 (custom_kernel.cpp:57-112, called from jit_compiler.py:41-45 for
// tensors that live on the host).  These are the reference's own entry points for CPU tensors, kept as what
// they are: a separate call for host tensors, single-threaded, in the tensors' dtype.  Nothing on
// the GPU path reaches them (every GPU entry point refuses a CPU tensor and these refuse a GPU
// tensor), and they share no code with the test oracle.
//   inputs = {gates [T], indices int32 [T], locations int32 [T], rows [T, hidden], slots [E * capacity, hidden]},
//   extra = {samples, hidden, capacity};  kernel_type 0: slots += gate * row (the caller zeroes slots),
//   1: rows = gate * slot row, zero rows for pairs without a slot,  2: gates = <slot row, row> or 0.
// A pair has a slot when index >= 0 and location < capacity (the reference's test, kept to the letter).
namespace {

template <typename T>
struct HostPair {                       // one choice plane laid over host memory
    T *gates; const int32_t *index; const int32_t *location; T *rows; T *slots;
    int64_t hidden, capacity;
    T *row(int64_t t) const { return rows + t * hidden; }
    T *slot(int64_t t) const
    {
        if (index[t] < 0 || location[t] >= capacity) return nullptr;
        return slots + ((int64_t)index[t] * capacity + location[t]) * hidden;
    }
};

template <typename T>
void host_scatter(const HostPair<T> &p, int64_t samples)
{
    for (int64_t t = 0; t < samples; ++t)
        if (T *dst = p.slot(t)) {
            const T g = p.gates[t], *src = p.row(t);
            for (int64_t j = 0; j < p.hidden; ++j) dst[j] += g * src[j];
        }
}

template <typename T>
void host_gather(const HostPair<T> &p, int64_t samples)
{
    for (int64_t t = 0; t < samples; ++t) {
        T *dst = p.row(t);
        if (const T *src = p.slot(t)) {
            const T g = p.gates[t];
            for (int64_t j = 0; j < p.hidden; ++j) dst[j] = g * src[j];
        } else {
            std::fill(dst, dst + p.hidden, T(0));
        }
    }
}

template <typename T>
void host_gate_gradient(const HostPair<T> &p, int64_t samples)
{
    for (int64_t t = 0; t < samples; ++t) {
        T sum = 0;                                              // summed in the tensors' dtype, left to right
        if (const T *a = p.slot(t)) {
            const T *b = p.row(t);
            for (int64_t j = 0; j < p.hidden; ++j) sum += a[j] * b[j];
        }
        p.gates[t] = sum;
    }
}

template <typename T>
void invoke_cpu(const std::vector<torch::Tensor> &ts, const std::vector<int> &extra, int kernel_type)
{
    const auto want = c10::CppTypeToScalarType<T>::value;
    AT_ASSERTM(ts.size() >= 5 && extra.size() >= 3, "invoke_cpu: expects 5 tensors and {samples, hidden, capacity}");
    for (size_t i = 0; i < ts.size(); ++i) {
        AT_ASSERTM(!ts[i].is_cuda(), "invoke_cpu: tensor must be a CPU tensor (GPU tensors take the GPU entry points)");
        AT_ASSERTM(ts[i].is_contiguous(), "invoke_cpu: tensor must be contiguous");
    }
    AT_ASSERTM(ts[0].scalar_type() == want && ts[3].scalar_type() == want && ts[4].scalar_type() == want,
               "invoke_cpu: gates, rows and slots must have the dtype of the entry point");
    AT_ASSERTM(ts[1].scalar_type() == at::kInt && ts[2].scalar_type() == at::kInt, "invoke_cpu: indices and locations must be int32");
    const int64_t samples = extra[0], hidden = extra[1], capacity = extra[2];
    AT_ASSERTM(samples >= 0 && hidden >= 0 && capacity >= 0, "invoke_cpu: negative size");
    AT_ASSERTM(ts[0].numel() >= samples && ts[1].numel() >= samples && ts[2].numel() >= samples &&
                   ts[3].numel() >= samples * hidden, "invoke_cpu: tensors smaller than {samples, hidden} say");
    const HostPair<T> p{ts[0].data_ptr<T>(), ts[1].data_ptr<int32_t>(), ts[2].data_ptr<int32_t>(), ts[3].data_ptr<T>(),
                        ts[4].data_ptr<T>(), hidden, capacity};
    // every slot a live pair names must lie inside the slots tensor
    for (int64_t t = 0; t < samples; ++t)
        if (p.index[t] >= 0 && p.location[t] < capacity)
            AT_ASSERTM(p.location[t] >= 0 && ((int64_t)p.index[t] * capacity + p.location[t] + 1) * hidden <= ts[4].numel(),
                       "invoke_cpu: a pair addresses a slot outside the slots tensor");
    if (kernel_type == 0) host_scatter(p, samples);
    else if (kernel_type == 1) host_gather(p, samples);
    else host_gate_gradient(p, samples);
}

} // namespace

torch::Tensor warp_cumsum(torch::Tensor x)
{
    CHECK_GPU(x);
    AT_ASSERTM(x.dim() == 2, "CHECK_EQ fails.");
    x = x.to(torch::kInt32).contiguous();
    auto y = torch::empty_like(x);
    const int T = (int)x.size(0), E = (int)x.size(1);
    auto ws = torch::empty({(int64_t)planmoe_cumsum_workspace_bytes(T, E)}, x.options().dtype(at::kByte));
    PM_CALL(planmoe_cumsum_sub_one((const int32_t *)x.data_ptr(), (int32_t *)y.data_ptr(), T, E, ws.data_ptr(),
                                   (size_t)ws.numel(), current_stream()));
    return y;
}

// the reference's NVRTC entry points (custom_kernel.cpp:295-298, jit.h): the mechanism this build
// replaces with compiled gfx950 kernels behind typed entry points
static void jit_unavailable(const char *what)
{
    AT_ASSERTM(false, what, ": this build has no run-time kernel compiler; its kernels are compiled into "
               "libplanmoe_hip.so (see include/planmoe_hip.h for the typed entry points)");
}
static void update_sdk_home(const torch::Tensor &) { jit_unavailable("update_sdk_home"); }
static int inject_source(const std::string &) { jit_unavailable("inject_source"); return -1; }
static void invoke(const std::vector<torch::Tensor> &, const std::vector<long> &, int) { jit_unavailable("invoke"); }

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m)
{
    m.def("update_sdk_home", &update_sdk_home, "not available in this build");
    m.def("invoke", &invoke, "not available in this build");
    m.def("inject_source", &inject_source, "not available in this build");
    m.def("registered_compressors", &planmoe::registered_compressors, "names of the compressor plug-ins registered from C++");
    m.def("invoke_cpu_fp32", &invoke_cpu<float>, "Invoke for Sparse Ops (CPU)");
    m.def("invoke_cpu_fp64", &invoke_cpu<double>, "Invoke for Sparse Ops (CPU)");
    m.def("compress_operation", &compress_operation, "Compress Operation");
    m.def("comm_operation", &comm_operation, "Comm Operation");
    m.def("decompress_operation", &decompress_operation, "Decompress Operation");
    m.def("clear_ptr_lst", &clear_ptr_lst, "Clear Ptr Lst");
}

TORCH_LIBRARY(tutel_ops, m) { m.def("cumsum", warp_cumsum); }
