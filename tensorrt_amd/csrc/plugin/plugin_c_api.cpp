// Flat C functions over the IPluginV3 objects (declared in trtamd_plugin_c.h).  Every function
// forwards to one interface method; the only logic here is converting descriptors and evaluating
// the dimension expressions a plugin builds in getOutputShapes.
#include "plugin_base.h"
#include "trtamd_plugin_c.h"

#include <deque>
#include <mutex>

namespace trtamd
{
namespace plugin
{
namespace
{

static_assert(sizeof(trtamd_plugin_field) == sizeof(PluginField), "PluginField layout");
static_assert(TRTAMD_MAX_DIMS == Dims::MAX_DIMS, "Dims::MAX_DIMS");

// ---- constant-folding expression builder ------------------------------------------------------------
// TensorRT's builder keeps dimension expressions symbolic; for a host that already knows every input
// extent, folding constants is the same computation.

class ConstExprImpl final : public apiv::VDimensionExpr
{
public:
    explicit ConstExprImpl(int64_t v)
        : value(v)
    {
    }
    bool isConstant() const override
    {
        return true;
    }
    int64_t getConstantValue() const override
    {
        return value;
    }
    bool isSizeTensor() const override
    {
        return false;
    }
    int64_t value;
};

class ConstExpr final : public IDimensionExpr
{
public:
    explicit ConstExpr(int64_t v)
        : impl(v)
    {
        mImpl = &impl;
    }
    ~ConstExpr() noexcept override = default;
    ConstExprImpl impl;
};

class FoldingBuilder final : public IExprBuilder, private apiv::VExprBuilder
{
public:
    FoldingBuilder()
    {
        mImpl = this;
    }
    ~FoldingBuilder() noexcept override = default;

private:
    IDimensionExpr const* constant(int64_t value) override
    {
        mPool.emplace_back(value);
        return &mPool.back();
    }
    IDimensionExpr const* operation(
        DimensionOperation op, IDimensionExpr const& first, IDimensionExpr const& second) override
    {
        int64_t const a = first.getConstantValue();
        int64_t const b = second.getConstantValue();
        auto floorDiv = [](int64_t x, int64_t y) {
            int64_t q = x / y;
            return (x % y != 0 && ((x < 0) != (y < 0))) ? q - 1 : q;
        };
        int64_t r = 0;
        switch (op)
        {
        case DimensionOperation::kSUM: r = a + b; break;
        case DimensionOperation::kPROD: r = a * b; break;
        case DimensionOperation::kMAX: r = a > b ? a : b; break;
        case DimensionOperation::kMIN: r = a < b ? a : b; break;
        case DimensionOperation::kSUB: r = a - b; break;
        case DimensionOperation::kEQUAL: r = a == b ? 1 : 0; break;
        case DimensionOperation::kLESS: r = a < b ? 1 : 0; break;
        case DimensionOperation::kFLOOR_DIV:
            if (b == 0)
            {
                return nullptr;
            }
            r = floorDiv(a, b);
            break;
        case DimensionOperation::kCEIL_DIV:
            if (b == 0)
            {
                return nullptr;
            }
            r = -floorDiv(-a, b);
            break;
        }
        return constant(r);
    }
    IDimensionExpr const* declareSizeTensor(int32_t, IDimensionExpr const& opt, IDimensionExpr const&) override
    {
        return &opt;
    }
    std::deque<ConstExpr> mPool; // deque: stable addresses
};

Dims toDims(int32_t nb, int64_t const* d)
{
    Dims out{};
    out.nbDims = nb;
    for (int32_t i = 0; i < Dims::MAX_DIMS; ++i)
    {
        out.d[i] = i < nb ? d[i] : 0;
    }
    return out;
}

PluginTensorDesc toDesc(trtamd_tensor_desc const& t)
{
    PluginTensorDesc d{};
    d.dims = toDims(t.nb_dims, t.dims);
    d.type = static_cast<DataType>(t.type);
    d.format = static_cast<TensorFormat>(t.format);
    d.scale = t.scale;
    return d;
}

std::vector<PluginTensorDesc> toDescs(trtamd_tensor_desc const* t, int32_t n)
{
    std::vector<PluginTensorDesc> v;
    for (int32_t i = 0; i < n; ++i)
    {
        v.push_back(toDesc(t[i]));
    }
    return v;
}

std::vector<DynamicPluginTensorDesc> toDynDescs(trtamd_tensor_desc const* t, int32_t n)
{
    std::vector<DynamicPluginTensorDesc> v;
    for (int32_t i = 0; i < n; ++i)
    {
        DynamicPluginTensorDesc d{};
        d.desc = toDesc(t[i]);
        d.min = toDims(t[i].nb_dims, t[i].min);
        d.max = toDims(t[i].nb_dims, t[i].max);
        d.opt = toDims(t[i].nb_dims, t[i].opt);
        v.push_back(d);
    }
    return v;
}

template <typename T>
T* capability(trtamd_plugin_t plugin, PluginCapabilityType type)
{
    if (!plugin)
    {
        return nullptr;
    }
    auto* p = static_cast<IPluginV3*>(plugin);
    return static_cast<T*>(p->getCapabilityInterface(type));
}

IPluginV3OneCore* core(trtamd_plugin_t p)
{
    return capability<IPluginV3OneCore>(p, PluginCapabilityType::kCORE);
}
IPluginV3OneBuild* build(trtamd_plugin_t p)
{
    return capability<IPluginV3OneBuild>(p, PluginCapabilityType::kBUILD);
}
IPluginV3OneRuntime* runtime(trtamd_plugin_t p)
{
    return capability<IPluginV3OneRuntime>(p, PluginCapabilityType::kRUNTIME);
}

class CaptureLogger final : public ILogger
{
public:
    void log(Severity severity, AsciiChar const* msg) noexcept override
    {
        if (severity <= Severity::kERROR)
        {
            std::lock_guard<std::mutex> lock(mMutex);
            mLast = msg ? msg : "";
        }
    }
    std::string take()
    {
        std::lock_guard<std::mutex> lock(mMutex);
        std::string s;
        s.swap(mLast);
        return s;
    }

private:
    std::mutex mMutex;
    std::string mLast;
};

CaptureLogger& captureLogger()
{
    static CaptureLogger* logger = new CaptureLogger();
    return *logger;
}

bool isKind(IPluginCreatorInterface* c, char const* kind)
{
    InterfaceInfo const info = c->getInterfaceInfo();
    return info.kind && std::string(info.kind) == kind;
}

IPluginCreatorInterface* creatorAt(int32_t index)
{
    int32_t n = 0;
    IPluginCreatorInterface* const* list = getPluginRegistry()->getAllCreators(&n);
    if (index < 0 || index >= n)
    {
        return nullptr;
    }
    return list[index];
}

IPluginV2DynamicExt* legacy(trtamd_legacy_plugin_t p)
{
    return static_cast<IPluginV2DynamicExt*>(p);
}

} // namespace
} // namespace plugin
} // namespace trtamd

using namespace trtamd::plugin;

extern "C" {

trtamd_creator_t trtamd_plugin_get_creator(char const* name, char const* version, char const* ns)
{
    IPluginCreatorInterface* c = getPluginRegistry()->getCreator(name, version, ns ? ns : "");
    return c && isKind(c, "PLUGIN CREATOR_V3ONE") ? static_cast<IPluginCreatorV3One*>(c) : nullptr;
}

int32_t trtamd_plugin_num_creators(void)
{
    int32_t n = 0;
    getPluginRegistry()->getAllCreators(&n);
    return n;
}

char const* trtamd_plugin_creator_name(int32_t index)
{
    auto* c = creatorAt(index);
    if (!c)
    {
        return nullptr;
    }
    return isKind(c, "PLUGIN CREATOR_V1") ? static_cast<IPluginCreator*>(c)->getPluginName()
                                           : static_cast<IPluginCreatorV3One*>(c)->getPluginName();
}

char const* trtamd_plugin_creator_version(int32_t index)
{
    auto* c = creatorAt(index);
    if (!c)
    {
        return nullptr;
    }
    return isKind(c, "PLUGIN CREATOR_V1") ? static_cast<IPluginCreator*>(c)->getPluginVersion()
                                           : static_cast<IPluginCreatorV3One*>(c)->getPluginVersion();
}

int32_t trtamd_plugin_creator_field_names(trtamd_creator_t creator, trtamd_plugin_field const** fields)
{
    if (!creator)
    {
        return -1;
    }
    PluginFieldCollection const* fc = static_cast<IPluginCreatorV3One*>(creator)->getFieldNames();
    if (!fc)
    {
        return -1;
    }
    if (fields)
    {
        *fields = reinterpret_cast<trtamd_plugin_field const*>(fc->fields);
    }
    return fc->nbFields;
}

trtamd_plugin_t trtamd_plugin_create(trtamd_creator_t creator, char const* layer_name,
    trtamd_plugin_field const* fields, int32_t nb_fields, int32_t phase)
{
    if (!creator)
    {
        return nullptr;
    }
    PluginFieldCollection fc{};
    fc.nbFields = nb_fields;
    fc.fields = reinterpret_cast<PluginField const*>(fields);
    return static_cast<IPluginCreatorV3One*>(creator)->createPlugin(
        layer_name, &fc, static_cast<TensorRTPhase>(phase));
}

void trtamd_plugin_destroy(trtamd_plugin_t plugin)
{
    delete static_cast<IPluginV3*>(plugin);
}

trtamd_plugin_t trtamd_plugin_clone(trtamd_plugin_t plugin)
{
    return plugin ? static_cast<IPluginV3*>(plugin)->clone() : nullptr;
}

char const* trtamd_plugin_name(trtamd_plugin_t plugin)
{
    auto* c = core(plugin);
    return c ? c->getPluginName() : nullptr;
}

char const* trtamd_plugin_version(trtamd_plugin_t plugin)
{
    auto* c = core(plugin);
    return c ? c->getPluginVersion() : nullptr;
}

char const* trtamd_plugin_namespace(trtamd_plugin_t plugin)
{
    auto* c = core(plugin);
    return c ? c->getPluginNamespace() : nullptr;
}

int32_t trtamd_plugin_nb_outputs(trtamd_plugin_t plugin)
{
    auto* b = build(plugin);
    return b ? b->getNbOutputs() : -1;
}

int32_t trtamd_plugin_output_types(
    trtamd_plugin_t plugin, int32_t* out_types, int32_t nb_outputs, int32_t const* in_types, int32_t nb_inputs)
{
    auto* b = build(plugin);
    if (!b)
    {
        return -1;
    }
    return b->getOutputDataTypes(reinterpret_cast<DataType*>(out_types), nb_outputs,
        reinterpret_cast<DataType const*>(in_types), nb_inputs);
}

int32_t trtamd_plugin_output_shapes(trtamd_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc* out, int32_t nb_outputs)
{
    auto* b = build(plugin);
    if (!b || nb_inputs < 0 || nb_outputs < 0)
    {
        return -1;
    }
    FoldingBuilder builder;
    std::vector<DimsExprs> ins(static_cast<size_t>(nb_inputs));
    for (int32_t i = 0; i < nb_inputs; ++i)
    {
        ins[i].nbDims = in[i].nb_dims;
        for (int32_t k = 0; k < in[i].nb_dims && k < TRTAMD_MAX_DIMS; ++k)
        {
            ins[i].d[k] = static_cast<IExprBuilder&>(builder).constant(in[i].dims[k]);
        }
    }
    std::vector<DimsExprs> outs(static_cast<size_t>(nb_outputs));
    int32_t const status = b->getOutputShapes(
        ins.data(), nb_inputs, nullptr, 0, outs.data(), nb_outputs, builder);
    if (status != 0)
    {
        return status;
    }
    for (int32_t i = 0; i < nb_outputs; ++i)
    {
        out[i].nb_dims = outs[i].nbDims;
        for (int32_t k = 0; k < outs[i].nbDims && k < TRTAMD_MAX_DIMS; ++k)
        {
            if (!outs[i].d[k])
            {
                return -1;
            }
            out[i].dims[k] = outs[i].d[k]->getConstantValue();
        }
    }
    return 0;
}

int32_t trtamd_plugin_supports_format(
    trtamd_plugin_t plugin, int32_t pos, trtamd_tensor_desc const* in_out, int32_t nb_inputs, int32_t nb_outputs)
{
    auto* b = build(plugin);
    if (!b)
    {
        return 0;
    }
    auto descs = toDynDescs(in_out, nb_inputs + nb_outputs);
    return b->supportsFormatCombination(pos, descs.data(), nb_inputs, nb_outputs) ? 1 : 0;
}

int32_t trtamd_plugin_configure(trtamd_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs)
{
    auto* b = build(plugin);
    if (!b)
    {
        return -1;
    }
    auto i = toDynDescs(in, nb_inputs);
    auto o = toDynDescs(out, nb_outputs);
    return b->configurePlugin(i.data(), nb_inputs, o.data(), nb_outputs);
}

size_t trtamd_plugin_workspace_size(trtamd_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs)
{
    auto* b = build(plugin);
    if (!b)
    {
        return 0;
    }
    auto i = toDynDescs(in, nb_inputs);
    auto o = toDynDescs(out, nb_outputs);
    return b->getWorkspaceSize(i.data(), nb_inputs, o.data(), nb_outputs);
}

int32_t trtamd_plugin_on_shape_change(trtamd_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs)
{
    auto* r = runtime(plugin);
    if (!r)
    {
        return -1;
    }
    auto i = toDescs(in, nb_inputs);
    auto o = toDescs(out, nb_outputs);
    return r->onShapeChange(i.data(), nb_inputs, o.data(), nb_outputs);
}

int32_t trtamd_plugin_enqueue(trtamd_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs, void const* const* inputs, void* const* outputs,
    void* workspace, void* stream)
{
    auto* r = runtime(plugin);
    if (!r)
    {
        return -1;
    }
    auto i = toDescs(in, nb_inputs);
    auto o = toDescs(out, nb_outputs);
    return r->enqueue(i.data(), o.data(), inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}

int32_t trtamd_plugin_fields_to_serialize(trtamd_plugin_t plugin, trtamd_plugin_field const** fields)
{
    auto* r = runtime(plugin);
    if (!r)
    {
        return -1;
    }
    PluginFieldCollection const* fc = r->getFieldsToSerialize();
    if (!fc)
    {
        return -1;
    }
    if (fields)
    {
        *fields = reinterpret_cast<trtamd_plugin_field const*>(fc->fields);
    }
    return fc->nbFields;
}

// ---- IPluginCreator / IPluginV2DynamicExt -----------------------------------------------------------

trtamd_legacy_creator_t trtamd_legacy_get_creator(char const* name, char const* version, char const* ns)
{
    IPluginCreatorInterface* c = getPluginRegistry()->getCreator(name, version, ns ? ns : "");
    return c && isKind(c, "PLUGIN CREATOR_V1") ? static_cast<IPluginCreator*>(c) : nullptr;
}

int32_t trtamd_legacy_creator_field_names(trtamd_legacy_creator_t creator, trtamd_plugin_field const** fields)
{
    if (!creator)
    {
        return -1;
    }
    PluginFieldCollection const* fc = static_cast<IPluginCreator*>(creator)->getFieldNames();
    if (!fc)
    {
        return -1;
    }
    if (fields)
    {
        *fields = reinterpret_cast<trtamd_plugin_field const*>(fc->fields);
    }
    return fc->nbFields;
}

trtamd_legacy_plugin_t trtamd_legacy_create(
    trtamd_legacy_creator_t creator, char const* layer_name, trtamd_plugin_field const* fields, int32_t nb_fields)
{
    if (!creator)
    {
        return nullptr;
    }
    PluginFieldCollection fc{};
    fc.nbFields = nb_fields;
    fc.fields = reinterpret_cast<PluginField const*>(fields);
    return static_cast<IPluginV2DynamicExt*>(static_cast<IPluginCreator*>(creator)->createPlugin(layer_name, &fc));
}

trtamd_legacy_plugin_t trtamd_legacy_deserialize(
    trtamd_legacy_creator_t creator, char const* layer_name, void const* data, size_t length)
{
    if (!creator)
    {
        return nullptr;
    }
    return static_cast<IPluginV2DynamicExt*>(
        static_cast<IPluginCreator*>(creator)->deserializePlugin(layer_name, data, length));
}

void trtamd_legacy_destroy(trtamd_legacy_plugin_t plugin)
{
    if (plugin)
    {
        legacy(plugin)->destroy();
    }
}

trtamd_legacy_plugin_t trtamd_legacy_clone(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->clone() : nullptr;
}

char const* trtamd_legacy_type(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->getPluginType() : nullptr;
}

char const* trtamd_legacy_version(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->getPluginVersion() : nullptr;
}

int32_t trtamd_legacy_nb_outputs(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->getNbOutputs() : -1;
}

int32_t trtamd_legacy_tensorrt_version(trtamd_legacy_plugin_t plugin)
{
    return plugin ? static_cast<IPluginV2*>(legacy(plugin))->getTensorRTVersion() : -1;
}

int32_t trtamd_legacy_initialize(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->initialize() : -1;
}

void trtamd_legacy_terminate(trtamd_legacy_plugin_t plugin)
{
    if (plugin)
    {
        legacy(plugin)->terminate();
    }
}

size_t trtamd_legacy_serialization_size(trtamd_legacy_plugin_t plugin)
{
    return plugin ? legacy(plugin)->getSerializationSize() : 0;
}

void trtamd_legacy_serialize(trtamd_legacy_plugin_t plugin, void* buffer)
{
    if (plugin)
    {
        legacy(plugin)->serialize(buffer);
    }
}

int32_t trtamd_legacy_output_type(trtamd_legacy_plugin_t plugin, int32_t index, int32_t const* in_types, int32_t nb_inputs)
{
    if (!plugin)
    {
        return -1;
    }
    std::vector<DataType> in(static_cast<size_t>(nb_inputs > 0 ? nb_inputs : 0));
    for (int32_t i = 0; i < nb_inputs; ++i)
    {
        in[i] = static_cast<DataType>(in_types[i]);
    }
    return static_cast<int32_t>(legacy(plugin)->getOutputDataType(index, in.data(), nb_inputs));
}

int32_t trtamd_legacy_output_dims(trtamd_legacy_plugin_t plugin, int32_t index, trtamd_tensor_desc const* in,
    int32_t nb_inputs, trtamd_tensor_desc* out)
{
    if (!plugin || nb_inputs < 0 || !out)
    {
        return -1;
    }
    FoldingBuilder builder;
    std::vector<DimsExprs> ins(static_cast<size_t>(nb_inputs));
    for (int32_t i = 0; i < nb_inputs; ++i)
    {
        ins[i].nbDims = in[i].nb_dims;
        for (int32_t k = 0; k < in[i].nb_dims && k < TRTAMD_MAX_DIMS; ++k)
        {
            ins[i].d[k] = static_cast<IExprBuilder&>(builder).constant(in[i].dims[k]);
        }
    }
    DimsExprs const d = legacy(plugin)->getOutputDimensions(index, ins.data(), nb_inputs, builder);
    if (d.nbDims < 0)
    {
        return -1;
    }
    out->nb_dims = d.nbDims;
    for (int32_t k = 0; k < d.nbDims && k < TRTAMD_MAX_DIMS; ++k)
    {
        if (!d.d[k])
        {
            return -1;
        }
        out->dims[k] = d.d[k]->getConstantValue();
    }
    return 0;
}

int32_t trtamd_legacy_supports_format(
    trtamd_legacy_plugin_t plugin, int32_t pos, trtamd_tensor_desc const* in_out, int32_t nb_inputs, int32_t nb_outputs)
{
    if (!plugin)
    {
        return 0;
    }
    auto v = toDescs(in_out, nb_inputs + nb_outputs);
    return legacy(plugin)->supportsFormatCombination(pos, v.data(), nb_inputs, nb_outputs) ? 1 : 0;
}

void trtamd_legacy_configure(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs)
{
    if (plugin)
    {
        auto i = toDynDescs(in, nb_inputs);
        auto o = toDynDescs(out, nb_outputs);
        legacy(plugin)->configurePlugin(i.data(), nb_inputs, o.data(), nb_outputs);
    }
}

size_t trtamd_legacy_workspace_size(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs)
{
    if (!plugin)
    {
        return 0;
    }
    auto i = toDescs(in, nb_inputs);
    auto o = toDescs(out, nb_outputs);
    return legacy(plugin)->getWorkspaceSize(i.data(), nb_inputs, o.data(), nb_outputs);
}

int32_t trtamd_legacy_enqueue(trtamd_legacy_plugin_t plugin, trtamd_tensor_desc const* in, int32_t nb_inputs,
    trtamd_tensor_desc const* out, int32_t nb_outputs, void const* const* inputs, void* const* outputs, void* workspace,
    void* stream)
{
    if (!plugin)
    {
        return -1;
    }
    auto i = toDescs(in, nb_inputs);
    auto o = toDescs(out, nb_outputs);
    return legacy(plugin)->enqueue(i.data(), o.data(), inputs, outputs, workspace, static_cast<hipStream_t>(stream));
}

void trtamd_plugin_capture_log(int32_t enable)
{
    if (enable)
    {
        initLibNvInferPlugins(static_cast<ILogger*>(&captureLogger()), "");
    }
    else if (currentLogger() == &captureLogger())
    {
        setLogger(nullptr);
    }
}

char const* trtamd_plugin_last_log(void)
{
    static thread_local std::string held;
    held = captureLogger().take();
    return held.c_str();
}

} // extern "C"
