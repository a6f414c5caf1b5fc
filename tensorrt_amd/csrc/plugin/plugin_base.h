// Common skeleton of the nine IPluginV3 classes.
//
// The reference spells out the IPluginV3 / IPluginV3OneCore / IPluginV3OneBuild /
// IPluginV3OneRuntime boilerplate in every plugin.  Here it lives once: the interface methods
// (noexcept, try/catch, log, failure value) are final in this base and forward to a handful of
// hooks that are allowed to throw.  A concrete plugin is its constructor, its hooks and a creator.
#pragma once

#include "plugin_common.h"

namespace trtamd
{
namespace plugin
{

class BertPluginBase : public IPluginV3,
                       public IPluginV3OneCore,
                       public IPluginV3OneBuild,
                       public IPluginV3OneRuntime
{
public:
    BertPluginBase(std::string layerName, char const* pluginName, char const* pluginVersion, int32_t nbInputs,
        int32_t nbOutputs);
    ~BertPluginBase() override = default;

    // IPluginV3
    IPluginCapability* getCapabilityInterface(PluginCapabilityType type) noexcept final;
    IPluginV3* clone() noexcept final;

    // IPluginV3OneCore
    char const* getPluginName() const noexcept final;
    char const* getPluginVersion() const noexcept final;
    char const* getPluginNamespace() const noexcept final;
    void setPluginNamespace(char const* ns) noexcept;

    // IPluginV3OneBuild
    int32_t configurePlugin(DynamicPluginTensorDesc const* in, int32_t nbInputs, DynamicPluginTensorDesc const* out,
        int32_t nbOutputs) noexcept final;
    int32_t getOutputDataTypes(
        DataType* outputTypes, int32_t nbOutputs, DataType const* inputTypes, int32_t nbInputs) const noexcept final;
    int32_t getOutputShapes(DimsExprs const* inputs, int32_t nbInputs, DimsExprs const* shapeInputs,
        int32_t nbShapeInputs, DimsExprs* outputs, int32_t nbOutputs, IExprBuilder& exprBuilder) noexcept final;
    bool supportsFormatCombination(
        int32_t pos, DynamicPluginTensorDesc const* inOut, int32_t nbInputs, int32_t nbOutputs) noexcept final;
    int32_t getNbOutputs() const noexcept final;
    size_t getWorkspaceSize(DynamicPluginTensorDesc const* inputs, int32_t nbInputs,
        DynamicPluginTensorDesc const* outputs, int32_t nbOutputs) const noexcept final;

    // IPluginV3OneRuntime
    int32_t onShapeChange(
        PluginTensorDesc const* in, int32_t nbInputs, PluginTensorDesc const* out, int32_t nbOutputs) noexcept final;
    int32_t enqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void* workspace, hipStream_t stream) noexcept final;
    IPluginV3* attachToContext(IPluginResourceContext* context) noexcept final;
    PluginFieldCollection const* getFieldsToSerialize() noexcept final;

protected:
    // ---- hooks (may throw) ----------------------------------------------------------------------
    virtual std::unique_ptr<BertPluginBase> doClone() = 0;
    virtual void doConfigure(DynamicPluginTensorDesc const* in, DynamicPluginTensorDesc const* out) {}
    virtual void doOutputTypes(DataType* outputTypes, DataType const* inputTypes) const = 0;
    virtual void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) = 0;
    virtual bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) = 0;
    virtual size_t doWorkspaceSize(DynamicPluginTensorDesc const* inputs, DynamicPluginTensorDesc const* outputs) const
    {
        return 0;
    }
    virtual void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const* out) {}
    virtual int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc,
        void const* const* inputs, void* const* outputs, void* workspace, hipStream_t stream)
        = 0;
    virtual void doSerialize(FieldList& fields) = 0;

    // number of inputs may depend on attributes (QKV plugins)
    virtual int32_t expectedInputs() const
    {
        return mNbInputs;
    }

    std::string const mLayerName;
    std::string mNamespace;
    char const* const mPluginName;
    char const* const mPluginVersion;
    int32_t const mNbInputs;
    int32_t const mNbOutputs;
    FieldList mSerialized;
};

// Creator skeleton: name/version/namespace, the advertised field list and the guarded createPlugin.
class BertCreatorBase : public IPluginCreatorV3One
{
public:
    BertCreatorBase(char const* pluginName, char const* pluginVersion, std::vector<PluginField> fields);

    IPluginV3* createPlugin(char const* name, PluginFieldCollection const* fc, TensorRTPhase phase) noexcept final;
    PluginFieldCollection const* getFieldNames() noexcept final;
    char const* getPluginName() const noexcept final;
    char const* getPluginVersion() const noexcept final;
    char const* getPluginNamespace() const noexcept final;
    void setPluginNamespace(char const* ns) noexcept;

protected:
    virtual std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc,
        TensorRTPhase phase)
        = 0;

private:
    char const* const mPluginName;
    char const* const mPluginVersion;
    std::string mNamespace;
    std::vector<PluginField> mFields;
    PluginFieldCollection mFC{};
};

// Every creator of this library, in registration order (for getCreators()).
void recordCreator(IPluginCreatorInterface* creator);
std::vector<IPluginCreatorInterface*> const& recordedCreators();

} // namespace plugin
} // namespace trtamd
