#include "plugin_base.h"

#include <mutex>

namespace trtamd
{
namespace plugin
{

BertPluginBase::BertPluginBase(std::string layerName, char const* pluginName, char const* pluginVersion,
    int32_t nbInputs, int32_t nbOutputs)
    : mLayerName(std::move(layerName))
    , mPluginName(pluginName)
    , mPluginVersion(pluginVersion)
    , mNbInputs(nbInputs)
    , mNbOutputs(nbOutputs)
{
}

IPluginCapability* BertPluginBase::getCapabilityInterface(PluginCapabilityType type) noexcept
{
    switch (type)
    {
    case PluginCapabilityType::kBUILD: return static_cast<IPluginV3OneBuild*>(this);
    case PluginCapabilityType::kRUNTIME: return static_cast<IPluginV3OneRuntime*>(this);
    case PluginCapabilityType::kCORE: return static_cast<IPluginV3OneCore*>(this);
    }
    logMessage(ILogger::Severity::kERROR, "getCapabilityInterface: unknown capability type");
    return nullptr;
}

IPluginV3* BertPluginBase::clone() noexcept
{
    try
    {
        auto p = doClone();
        p->setPluginNamespace(mNamespace.c_str());
        return p.release();
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return nullptr;
}

char const* BertPluginBase::getPluginName() const noexcept
{
    return mPluginName;
}

char const* BertPluginBase::getPluginVersion() const noexcept
{
    return mPluginVersion;
}

char const* BertPluginBase::getPluginNamespace() const noexcept
{
    return mNamespace.c_str();
}

void BertPluginBase::setPluginNamespace(char const* ns) noexcept
{
    try
    {
        mNamespace = ns ? ns : "";
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
}

int32_t BertPluginBase::configurePlugin(DynamicPluginTensorDesc const* in, int32_t nbInputs,
    DynamicPluginTensorDesc const* out, int32_t nbOutputs) noexcept
{
    try
    {
        TRTAMD_VALIDATE(in != nullptr && out != nullptr);
        TRTAMD_VALIDATE(nbInputs == expectedInputs());
        TRTAMD_VALIDATE(nbOutputs == mNbOutputs);
        doConfigure(in, out);
        return kSTATUS_SUCCESS;
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return kSTATUS_FAILURE;
}

int32_t BertPluginBase::getOutputDataTypes(
    DataType* outputTypes, int32_t nbOutputs, DataType const* inputTypes, int32_t nbInputs) const noexcept
{
    try
    {
        TRTAMD_VALIDATE(outputTypes != nullptr);
        TRTAMD_VALIDATE(inputTypes != nullptr);
        TRTAMD_VALIDATE(nbOutputs == mNbOutputs);
        TRTAMD_VALIDATE(nbInputs == expectedInputs());
        doOutputTypes(outputTypes, inputTypes);
        return kSTATUS_SUCCESS;
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return kSTATUS_FAILURE;
}

int32_t BertPluginBase::getOutputShapes(DimsExprs const* inputs, int32_t nbInputs, DimsExprs const* /*shapeInputs*/,
    int32_t nbShapeInputs, DimsExprs* outputs, int32_t nbOutputs, IExprBuilder& exprBuilder) noexcept
{
    try
    {
        TRTAMD_VALIDATE(inputs != nullptr);
        TRTAMD_VALIDATE(outputs != nullptr);
        TRTAMD_VALIDATE(nbInputs == expectedInputs());
        TRTAMD_VALIDATE(nbShapeInputs == 0);
        TRTAMD_VALIDATE(nbOutputs == mNbOutputs);
        doOutputShapes(inputs, outputs, exprBuilder);
        return kSTATUS_SUCCESS;
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return kSTATUS_FAILURE;
}

bool BertPluginBase::supportsFormatCombination(
    int32_t pos, DynamicPluginTensorDesc const* inOut, int32_t nbInputs, int32_t nbOutputs) noexcept
{
    try
    {
        TRTAMD_VALIDATE(inOut != nullptr);
        TRTAMD_VALIDATE(nbInputs == expectedInputs());
        TRTAMD_VALIDATE(nbOutputs == mNbOutputs);
        TRTAMD_VALIDATE(pos >= 0 && pos < nbInputs + nbOutputs);
        return doSupportsFormat(pos, inOut);
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return false;
}

int32_t BertPluginBase::getNbOutputs() const noexcept
{
    return mNbOutputs;
}

size_t BertPluginBase::getWorkspaceSize(DynamicPluginTensorDesc const* inputs, int32_t /*nbInputs*/,
    DynamicPluginTensorDesc const* outputs, int32_t /*nbOutputs*/) const noexcept
{
    try
    {
        return doWorkspaceSize(inputs, outputs);
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return 0;
}

int32_t BertPluginBase::onShapeChange(
    PluginTensorDesc const* in, int32_t nbInputs, PluginTensorDesc const* out, int32_t nbOutputs) noexcept
{
    try
    {
        TRTAMD_VALIDATE(in != nullptr);
        TRTAMD_VALIDATE(out != nullptr);
        TRTAMD_VALIDATE(nbInputs == expectedInputs());
        TRTAMD_VALIDATE(nbOutputs == mNbOutputs);
        doShapeChange(in, out);
        return kSTATUS_SUCCESS;
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return kSTATUS_FAILURE;
}

int32_t BertPluginBase::enqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc,
    void const* const* inputs, void* const* outputs, void* workspace, hipStream_t stream) noexcept
{
    try
    {
        TRTAMD_VALIDATE(inputDesc != nullptr && outputDesc != nullptr && inputs != nullptr && outputs != nullptr);
        return doEnqueue(inputDesc, outputDesc, inputs, outputs, workspace, stream);
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return -1;
}

IPluginV3* BertPluginBase::attachToContext(IPluginResourceContext* /*context*/) noexcept
{
    // Each execution context works on its own copy.  The reference attaches a per-context cuBLAS
    // handle here for the attention plugins; this library's kernels need no handle.
    return clone();
}

PluginFieldCollection const* BertPluginBase::getFieldsToSerialize() noexcept
{
    try
    {
        mSerialized.clear();
        doSerialize(mSerialized);
        return mSerialized.collection();
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return nullptr;
}

// ---- creator -----------------------------------------------------------------------------------

namespace
{
std::mutex gCreatorMutex;
std::vector<IPluginCreatorInterface*>& creatorList()
{
    static std::vector<IPluginCreatorInterface*> list;
    return list;
}
} // namespace

void recordCreator(IPluginCreatorInterface* creator)
{
    std::lock_guard<std::mutex> lock(gCreatorMutex);
    creatorList().push_back(creator);
}

std::vector<IPluginCreatorInterface*> const& recordedCreators()
{
    return creatorList();
}

BertCreatorBase::BertCreatorBase(char const* pluginName, char const* pluginVersion, std::vector<PluginField> fields)
    : mPluginName(pluginName)
    , mPluginVersion(pluginVersion)
    , mFields(std::move(fields))
{
    mFC.nbFields = static_cast<int32_t>(mFields.size());
    mFC.fields = mFields.data();
    recordCreator(this);
}

IPluginV3* BertCreatorBase::createPlugin(char const* name, PluginFieldCollection const* fc, TensorRTPhase phase) noexcept
{
    try
    {
        TRTAMD_VALIDATE_MSG(fc != nullptr, "Plugin Field collection is null");
        TRTAMD_VALIDATE_MSG(fc->nbFields == 0 || fc->fields != nullptr, "Plugin Fields are null");
        for (int32_t i = 0; i < fc->nbFields; ++i)
        {
            TRTAMD_VALIDATE(fc->fields[i].name != nullptr);
        }
        auto p = doCreate(name ? name : "", fc, phase);
        p->setPluginNamespace(mNamespace.c_str());
        return p.release();
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
    return nullptr;
}

PluginFieldCollection const* BertCreatorBase::getFieldNames() noexcept
{
    return &mFC;
}

char const* BertCreatorBase::getPluginName() const noexcept
{
    return mPluginName;
}

char const* BertCreatorBase::getPluginVersion() const noexcept
{
    return mPluginVersion;
}

char const* BertCreatorBase::getPluginNamespace() const noexcept
{
    return mNamespace.c_str();
}

void BertCreatorBase::setPluginNamespace(char const* ns) noexcept
{
    try
    {
        mNamespace = ns ? ns : "";
    }
    catch (std::exception const& e)
    {
        reportCaught(e);
    }
}

} // namespace plugin
} // namespace trtamd
