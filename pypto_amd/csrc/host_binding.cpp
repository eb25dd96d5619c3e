// pybind11 layer between the Python operators and the C ABI of libpypto_amd.so: torch tensors in, one C call out.
//
// Plays the role of the reference's LaunchKernelTorch (python/src/bindings/runtime.cpp:625-723) and of its tensor
// converter (python/src/bindings/torch_tensor_converter.cpp:91-214): every operand must be a dense torch.Tensor (no
// DTensor), all on one HIP device; the operands become a flat PtoTensorDesc list (address, DataType position, shape),
// the workspace comes from torch's caching allocator, and the launch goes to the caller's current HIP stream without
// waiting for it.  Nothing below this file sees a torch type: the C entry points of include/pypto_amd.h do all the
// operator-specific validation and launch the kernels.  Every operator's entry points share one machine-level
// signature (descriptor list, count, pointer to the operator's parameter block, ...), so they are held as addresses
// handed over by the Python side, which loads the library.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <cstring>
#include <string>
#include <vector>

#include "pypto_amd.h"

namespace {

using WorkspaceFn = uint64_t (*)(const PtoTensorDesc*, uint32_t, const void*);
using LaunchFn = int (*)(const PtoTensorDesc*, uint32_t, const void*, void*, uint64_t, void*, int);

struct Op {
    const char* name;
    size_t params_bytes;
    WorkspaceFn workspace; // bound to the loaded library's pto_<name>_workspace / pto_<name>_launch by bind()
    LaunchFn launch;
};

Op kOps[] = {
    {"sfa_quant", sizeof(PtoSfaParams)},
    {"sfa_antiquant", sizeof(PtoSfaParams)},
    {"lightning_indexer", sizeof(PtoIndexerParams)},
    {"select_experts", sizeof(PtoSelectExpertsParams)},
    {"gqa_decode", sizeof(PtoGqaParams)},
    {"indexer_prolog", sizeof(PtoIndexerPrologParams)},
    {"mla_prolog_quant", sizeof(PtoMlaPrologParams)},
    {"mla_indexer_prolog_quant", sizeof(PtoMlaIndexerPrologParams)},
    {"attention_pre_quant", sizeof(PtoAttentionPreQuantParams)},
    {"paged_gather", sizeof(PtoPagedGatherParams)},
    {"topk", sizeof(PtoTopkParams)},
};
constexpr int kNumOps = sizeof(kOps) / sizeof(kOps[0]);

// framework/include/tilefwk/data_type.h:33-65: positions in the reference's DataType enum
int dtype_code(at::ScalarType t)
{
    switch (t) {
    case at::kChar: return PTO_DT_INT8;
    case at::kInt: return PTO_DT_INT32;
    case at::kLong: return PTO_DT_INT64;
    case at::kHalf: return PTO_DT_FP16;
    case at::kFloat: return PTO_DT_FP32;
    case at::kBFloat16: return PTO_DT_BF16;
    default: return -1;
    }
}

// A failure of the binding's own checks (as opposed to a status of the C ABI): Python turns it into FeError as it is.
struct BindingError : std::runtime_error {
    using std::runtime_error::runtime_error;
};

struct Described {
    std::vector<PtoTensorDesc> descs; // (the caller's sequence keeps the operands alive until the launch has been queued)
    c10::Device device = c10::Device(c10::kCPU);
};

// The checks of the reference's binding, in its order and with its messages, and the descriptor list.
Described describe(const py::sequence& operands)
{
    Described d;
    const py::object fast = py::reinterpret_steal<py::object>(PySequence_Fast(operands.ptr(), "the operands must be a sequence"));
    if (!fast) throw py::error_already_set();
    const size_t n = (size_t)PySequence_Fast_GET_SIZE(fast.ptr());
    PyObject** items = PySequence_Fast_ITEMS(fast.ptr());
    d.descs.resize(n);
    for (size_t i = 0; i < n; ++i) {
        const py::handle o(items[i]);
        if (!THPVariable_Check(o.ptr())) {
            throw BindingError("Input " + std::to_string(i + 1) + " (index " + std::to_string(i) + ") must be a torch.Tensor, got " +
                                     std::string(py::str(py::type::of(o))));
        }
        if (!THPVariable_CheckExact(o.ptr()) && std::string(py::str(py::type::of(o).attr("__name__"))) == "DTensor") {
            throw BindingError("Input " + std::to_string(i + 1) + " (index " + std::to_string(i) + ") must not be a DTensor, got " +
                                     std::string(py::str(py::type::of(o))));
        }
        const at::Tensor& t = THPVariable_Unpack(o.ptr());
        if (!t.is_contiguous()) throw BindingError("not all tensors are contiguous");
        if (i == 0)
            d.device = t.device();
        else if (t.device() != d.device)
            throw BindingError("all tensors must be on the same device, got " + d.device.str() + " and " + t.device().str());
        const int code = dtype_code(t.scalar_type());
        if (code < 0) throw py::value_error(std::string("unsupported tensor dtype ") + c10::toString(t.scalar_type()));
        const int64_t r = t.dim();
        if (r > 8) throw py::value_error("tensors of more than 8 dimensions are not supported");
        PtoTensorDesc& desc = d.descs[i];
        desc.addr = t.numel() ? t.data_ptr() : nullptr; // (an empty tensor carries a null address)
        desc.dataType = code;
        desc.rank = (int32_t)r;
        for (int64_t k = 0; k < 8; ++k) desc.shape[k] = k < r ? t.size(k) : 0;
    }
    return d;
}

const char* (*g_last_error)() = nullptr;

const Op& op_of(int op)
{
    if (op < 0 || op >= kNumOps) throw py::value_error("unknown operator id " + std::to_string(op));
    if (kOps[op].launch == nullptr) throw std::runtime_error(std::string(kOps[op].name) + ": the C entry points are not bound");
    return kOps[op];
}

// Entry points of the library the Python side has loaded, by address: {operator: (pto_<op>_workspace, pto_<op>_launch)}
// and pto_last_error.  The library is loaded once, by path, in one place; this module does not link against it.
void bind(const py::dict& table, uintptr_t last_error)
{
    for (int i = 0; i < kNumOps; ++i) {
        if (!table.contains(kOps[i].name)) throw py::value_error(std::string("no entry points given for ") + kOps[i].name);
        const py::tuple pair = table[kOps[i].name];
        kOps[i].workspace = reinterpret_cast<WorkspaceFn>(pair[0].cast<uintptr_t>());
        kOps[i].launch = reinterpret_cast<LaunchFn>(pair[1].cast<uintptr_t>());
    }
    g_last_error = reinterpret_cast<const char* (*)()>(last_error);
}

const void* params_of(const Op& o, const py::bytes& params, std::string& storage)
{
    storage = params; // (a copy: the C side wants a properly aligned struct, and bytes objects are)
    if (storage.size() != o.params_bytes)
        throw py::value_error(std::string(o.name) + ": parameter block of " + std::to_string(storage.size()) + " bytes, expected " +
                              std::to_string(o.params_bytes));
    return storage.data();
}

[[noreturn]] void raise_status(int rc)
{
    const std::string msg = g_last_error ? g_last_error() : "";
    switch (rc) {
    case PTO_ERR_DTYPE:
    case PTO_ERR_SHAPE:
    case PTO_ERR_PARAM:
    case PTO_ERR_ALIGN: throw py::value_error(msg);
    default: throw std::runtime_error(msg);
    }
}

// Validate, size the workspace, launch on the current stream of the operands' device.  Returns the workspace size.
uint64_t launch(int op, const py::sequence& operands, const py::bytes& params)
{
    const Op& o = op_of(op);
    std::string pstore;
    const void* p = params_of(o, params, pstore);
    Described d = describe(operands);
    if (d.descs.empty()) throw BindingError(std::string(o.name) + ": no tensors");
    if (!d.device.is_cuda())
        throw BindingError("tensors must be on a HIP device (torch device type 'cuda'), got " + d.device.str());
    const uint32_t n = (uint32_t)d.descs.size();
    const c10::hip::HIPGuard guard(d.device.index());
    const uint64_t ws_bytes = o.workspace(d.descs.data(), n, p);
    at::Tensor ws;
    void* ws_ptr = nullptr;
    if (ws_bytes) {
        ws = at::empty({(int64_t)ws_bytes}, at::TensorOptions().dtype(at::kByte).device(d.device));
        ws_ptr = ws.data_ptr();
    }
    // (the caching allocator hands the workspace's memory out again only to work queued later on this same stream)
    hipStream_t stream = c10::hip::getCurrentHIPStream(d.device.index()).stream();
    const int rc = o.launch(d.descs.data(), n, p, ws_ptr, ws_bytes, stream, 0);
    if (rc != PTO_OK) raise_status(rc);
    return ws_bytes;
}

// The descriptor list as bytes, and the operands' device as a string: the validation half of launch(), callable without a GPU.
py::tuple describe_py(const py::sequence& operands)
{
    Described d = describe(operands);
    return py::make_tuple(py::bytes(reinterpret_cast<const char*>(d.descs.data()), d.descs.size() * sizeof(PtoTensorDesc)),
                          d.descs.empty() ? std::string() : d.device.str());
}

} // namespace

PYBIND11_MODULE(_host, m)
{
    m.doc() = "torch tensors -> C ABI of libpypto_amd.so";
    py::register_exception<BindingError>(m, "BindingError", PyExc_RuntimeError);
    m.def("launch", &launch, py::arg("op"), py::arg("tensors"), py::arg("params"));
    m.def("describe", &describe_py, py::arg("tensors"));
    m.def("bind", &bind, py::arg("entry_points"), py::arg("last_error"));
    m.attr("ABI_VERSION") = 2; // the version of include/pypto_amd.h this file was written against
    py::dict ids;
    for (int i = 0; i < kNumOps; ++i) ids[kOps[i].name] = i;
    m.attr("OPS") = ids;
    py::dict sizes;
    for (int i = 0; i < kNumOps; ++i) sizes[kOps[i].name] = kOps[i].params_bytes;
    m.attr("PARAM_BYTES") = sizes;
}
