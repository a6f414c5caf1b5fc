/*
 * The slice of the TensorRT plugin API that the BERT encoder plugins implement and an engine-side
 * caller uses to drive them, re-declared for a machine that has no TensorRT: same namespace,
 * names, enumerator values and virtual-function order as the reference headers, so plugin code
 * and callers stay source compatible and a vtable built against either header matches.
 *
 * Reference definitions (paths relative to the reference root):
 *   DataType, Dims64, InterfaceInfo, APILanguage, IVersionedInterface  include/NvInferRuntimeBase.h:148-307
 *   PluginFieldType, PluginField, PluginFieldCollection, TensorRTPhase,
 *   PluginCapabilityType, IPluginCapability, IPluginResource,
 *   IPluginCreatorInterface, IPluginV3                                 include/NvInferPluginBase.h:36-240
 *   PluginTensorDesc                                                   include/NvInferRuntimePlugin.h:72-83
 *   Weights, DimensionOperation, IDimensionExpr, IExprBuilder, DimsExprs,
 *   DynamicPluginTensorDesc, IPluginResourceContext, IPluginV3OneCore,
 *   IPluginV3OneBuild, IPluginV3OneRuntime, TensorFormat, ILogger,
 *   ILoggerFinder, IPluginCreatorV3One, PluginRegistrar,
 *   REGISTER_TENSORRT_PLUGIN, getPluginRegistry, getLogger              include/NvInferRuntime.h:120-374, 791-1176,
 *                                                                      1420-1622, 5044-5148, 5285-5305
 *   VDimensionExpr, VExprBuilder                                       include/NvInferImpl.h:232-264
 *   IPluginRegistry                                                    include/NvInferRuntimeCommon.h:55-249
 *   initLibNvInferPlugins                                              include/NvInferPlugin.h:29-40
 *   PluginVersion, PluginFormat, IPluginV2, IPluginV2Ext, IPluginCreator include/NvInferRuntimePlugin.h:54, 94-106,
 *                                                                      138-460, 473-660, 784-909
 *   IPluginV2DynamicExt                                                include/NvInferRuntime.h:406-570
 * The stream argument of enqueue() is a hipStream_t (an opaque pointer, like cudaStream_t).
 */
#ifndef TRTAMD_NVINFER_API_H
#define TRTAMD_NVINFER_API_H

#include <cstddef>
#include <cstdint>

#define NV_TENSORRT_MAJOR 11
#define NV_TENSORRT_MINOR 1
#define NV_TENSORRT_PATCH 0
#define NV_TENSORRT_BUILD 106
#define NV_TENSORRT_VERSION_INT(major, minor, patch) ((major) *10000L + (minor) *100L + (patch) *1L)
#define NV_TENSORRT_VERSION NV_TENSORRT_VERSION_INT(NV_TENSORRT_MAJOR, NV_TENSORRT_MINOR, NV_TENSORRT_PATCH)

#ifndef TENSORRTAPI
#define TENSORRTAPI __attribute__((visibility("default")))
#endif

struct ihipStream_t;
typedef ihipStream_t* hipStream_t;
// Source compatibility with callers written against the reference headers.
typedef hipStream_t cudaStream_t;

namespace nvinfer1
{

using AsciiChar = char;

enum class DataType : int32_t
{
    kFLOAT = 0,
    kHALF = 1,
    kINT8 = 2,
    kINT32 = 3,
    kBOOL = 4,
    kUINT8 = 5,
    kFP8 = 6,
    kBF16 = 7,
    kINT64 = 8,
    kINT4 = 9,
    kFP4 = 10,
    kE8M0 = 11
};

class Dims64
{
public:
    static constexpr int32_t MAX_DIMS{8};
    int32_t nbDims;
    int64_t d[MAX_DIMS];
};
using Dims = Dims64;

using InterfaceKind = char const*;

class InterfaceInfo
{
public:
    InterfaceKind kind;
    int32_t major;
    int32_t minor;
};

enum class APILanguage : int32_t
{
    kCPP = 0,
    kPYTHON = 1
};

class IVersionedInterface
{
public:
    virtual APILanguage getAPILanguage() const noexcept
    {
        return APILanguage::kCPP;
    }
    virtual InterfaceInfo getInterfaceInfo() const noexcept = 0;
    virtual ~IVersionedInterface() noexcept = default;

protected:
    IVersionedInterface() = default;
    IVersionedInterface(IVersionedInterface const&) = default;
    IVersionedInterface(IVersionedInterface&&) = default;
    IVersionedInterface& operator=(IVersionedInterface const&) & = default;
    IVersionedInterface& operator=(IVersionedInterface&&) & = default;
};

enum class TensorFormat : int32_t
{
    kLINEAR = 0,
    kCHW2 = 1,
    kHWC8 = 2,
    kCHW4 = 3,
    kCHW16 = 4,
    kCHW32 = 5,
    kDHWC8 = 6,
    kCDHW32 = 7,
    kHWC = 8,
    kDLA_LINEAR = 9,
    kDLA_HWC4 = 10,
    kHWC16 = 11,
    kDHWC = 12
};

struct PluginTensorDesc
{
    Dims dims;
    DataType type;
    TensorFormat format;
    float scale;
};

struct DynamicPluginTensorDesc
{
    PluginTensorDesc desc;
    Dims min;
    Dims max;
    Dims opt;
};

class Weights
{
public:
    DataType type;
    void const* values;
    int64_t count;
};

enum class DimensionOperation : int32_t
{
    kSUM = 0,
    kPROD = 1,
    kMAX = 2,
    kMIN = 3,
    kSUB = 4,
    kEQUAL = 5,
    kLESS = 6,
    kFLOOR_DIV = 7,
    kCEIL_DIV = 8
};

class IDimensionExpr;

namespace apiv
{
class VRoot
{
public:
    virtual ~VRoot() noexcept = default;
};

class VDimensionExpr : public VRoot
{
public:
    virtual bool isConstant() const = 0;
    virtual int64_t getConstantValue() const = 0;
    virtual bool isSizeTensor() const = 0;
};

class VExprBuilder : public VRoot
{
public:
    virtual IDimensionExpr const* constant(int64_t value) = 0;
    virtual IDimensionExpr const* operation(
        DimensionOperation op, IDimensionExpr const& first, IDimensionExpr const& second)
        = 0;
    virtual IDimensionExpr const* declareSizeTensor(
        int32_t outputIndex, IDimensionExpr const& opt, IDimensionExpr const& upper)
        = 0;
};
} // namespace apiv

class INoCopy
{
protected:
    INoCopy() = default;
    virtual ~INoCopy() = default;
    INoCopy(INoCopy const& other) = delete;
    INoCopy& operator=(INoCopy const& other) = delete;
    INoCopy(INoCopy&& other) = delete;
    INoCopy& operator=(INoCopy&& other) = delete;
};

class IDimensionExpr : public INoCopy
{
public:
    bool isConstant() const noexcept
    {
        return mImpl->isConstant();
    }
    int64_t getConstantValue() const noexcept
    {
        return mImpl->getConstantValue();
    }

protected:
    apiv::VDimensionExpr* mImpl;
    virtual ~IDimensionExpr() noexcept = 0;

public:
    bool isSizeTensor() const noexcept
    {
        return mImpl->isSizeTensor();
    }
};
inline IDimensionExpr::~IDimensionExpr() noexcept = default;

class IExprBuilder : public INoCopy
{
public:
    IDimensionExpr const* constant(int64_t value) noexcept
    {
        return mImpl->constant(value);
    }
    IDimensionExpr const* operation(
        DimensionOperation op, IDimensionExpr const& first, IDimensionExpr const& second) noexcept
    {
        return mImpl->operation(op, first, second);
    }

protected:
    apiv::VExprBuilder* mImpl;
    virtual ~IExprBuilder() noexcept = 0;

public:
    IDimensionExpr const* declareSizeTensor(int32_t outputIndex, IDimensionExpr const& opt, IDimensionExpr const& upper)
    {
        return mImpl->declareSizeTensor(outputIndex, opt, upper);
    }
};
inline IExprBuilder::~IExprBuilder() noexcept = default;

class DimsExprs
{
public:
    int32_t nbDims;
    IDimensionExpr const* d[Dims::MAX_DIMS];
};

enum class PluginFieldType : int32_t
{
    kFLOAT16 = 0,
    kFLOAT32 = 1,
    kFLOAT64 = 2,
    kINT8 = 3,
    kINT16 = 4,
    kINT32 = 5,
    kCHAR = 6,
    kDIMS = 7,
    kUNKNOWN = 8,
    kBF16 = 9,
    kINT64 = 10,
    kFP8 = 11,
    kINT4 = 12,
    kFP4 = 13
};

class PluginField
{
public:
    AsciiChar const* name;
    void const* data;
    PluginFieldType type;
    int32_t length;

    PluginField(AsciiChar const* const name_ = nullptr, void const* const data_ = nullptr,
        PluginFieldType const type_ = PluginFieldType::kUNKNOWN, int32_t const length_ = 0) noexcept
        : name(name_)
        , data(data_)
        , type(type_)
        , length(length_)
    {
    }
};

struct PluginFieldCollection
{
    int32_t nbFields{};
    PluginField const* fields{};
};

enum class TensorRTPhase : int32_t
{
    kBUILD = 0,
    kRUNTIME = 1
};

enum class PluginCapabilityType : int32_t
{
    kCORE = 0,
    kBUILD = 1,
    kRUNTIME = 2
};

class IPluginCapability : public IVersionedInterface
{
};

class IPluginResource : public IVersionedInterface
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"IPluginResource", 1, 0};
    }
    virtual int32_t release() noexcept = 0;
    virtual IPluginResource* clone() noexcept = 0;
    ~IPluginResource() noexcept override = default;
    IPluginResource() = default;
};

class IPluginCreatorInterface : public IVersionedInterface
{
public:
    ~IPluginCreatorInterface() noexcept override = default;

protected:
    IPluginCreatorInterface() = default;
};

class IPluginV3 : public IVersionedInterface
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN", 1, 0};
    }
    virtual IPluginCapability* getCapabilityInterface(PluginCapabilityType type) noexcept = 0;
    virtual IPluginV3* clone() noexcept = 0;
};

class IGpuAllocator;
class IErrorRecorder;

class IPluginResourceContext
{
public:
    virtual IGpuAllocator* getGpuAllocator() const noexcept = 0;
    virtual IErrorRecorder* getErrorRecorder() const noexcept = 0;
    virtual ~IPluginResourceContext() noexcept = 0;

protected:
    IPluginResourceContext() = default;
};
inline IPluginResourceContext::~IPluginResourceContext() noexcept = default;

class IPluginV3OneCore : public IPluginCapability
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN_V3ONE_CORE", 1, 0};
    }
    virtual AsciiChar const* getPluginName() const noexcept = 0;
    virtual AsciiChar const* getPluginVersion() const noexcept = 0;
    virtual AsciiChar const* getPluginNamespace() const noexcept = 0;
};

class IPluginV3OneBuild : public IPluginCapability
{
public:
    static constexpr int32_t kDEFAULT_FORMAT_COMBINATION_LIMIT = 100;

    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN_V3ONE_BUILD", 1, 0};
    }
    virtual int32_t configurePlugin(DynamicPluginTensorDesc const* in, int32_t nbInputs,
        DynamicPluginTensorDesc const* out, int32_t nbOutputs) noexcept = 0;
    virtual int32_t getOutputDataTypes(
        DataType* outputTypes, int32_t nbOutputs, DataType const* inputTypes, int32_t nbInputs) const noexcept = 0;
    virtual int32_t getOutputShapes(DimsExprs const* inputs, int32_t nbInputs, DimsExprs const* shapeInputs,
        int32_t nbShapeInputs, DimsExprs* outputs, int32_t nbOutputs, IExprBuilder& exprBuilder) noexcept = 0;
    virtual bool supportsFormatCombination(
        int32_t pos, DynamicPluginTensorDesc const* inOut, int32_t nbInputs, int32_t nbOutputs) noexcept = 0;
    virtual int32_t getNbOutputs() const noexcept = 0;
    virtual size_t getWorkspaceSize(DynamicPluginTensorDesc const* /*inputs*/, int32_t /*nbInputs*/,
        DynamicPluginTensorDesc const* /*outputs*/, int32_t /*nbOutputs*/) const noexcept
    {
        return 0;
    }
    virtual int32_t getValidTactics(int32_t* /*tactics*/, int32_t /*nbTactics*/) noexcept
    {
        return 0;
    }
    virtual int32_t getNbTactics() noexcept
    {
        return 0;
    }
    virtual char const* getTimingCacheID() noexcept
    {
        return nullptr;
    }
    virtual int32_t getFormatCombinationLimit() noexcept
    {
        return kDEFAULT_FORMAT_COMBINATION_LIMIT;
    }
    virtual char const* getMetadataString() noexcept
    {
        return nullptr;
    }
};

class IPluginV3OneRuntime : public IPluginCapability
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN_V3ONE_RUNTIME", 1, 0};
    }
    virtual int32_t setTactic(int32_t /*tactic*/) noexcept
    {
        return 0;
    }
    virtual int32_t onShapeChange(
        PluginTensorDesc const* in, int32_t nbInputs, PluginTensorDesc const* out, int32_t nbOutputs) noexcept = 0;
    virtual int32_t enqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc,
        void const* const* inputs, void* const* outputs, void* workspace, hipStream_t stream) noexcept = 0;
    virtual IPluginV3* attachToContext(IPluginResourceContext* context) noexcept = 0;
    virtual PluginFieldCollection const* getFieldsToSerialize() noexcept = 0;
};

class IPluginCreatorV3One : public IPluginCreatorInterface
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN CREATOR_V3ONE", 1, 0};
    }
    virtual IPluginV3* createPlugin(
        AsciiChar const* name, PluginFieldCollection const* fc, TensorRTPhase phase) noexcept = 0;
    virtual PluginFieldCollection const* getFieldNames() noexcept = 0;
    virtual AsciiChar const* getPluginName() const noexcept = 0;
    virtual AsciiChar const* getPluginVersion() const noexcept = 0;
    virtual AsciiChar const* getPluginNamespace() const noexcept = 0;
    IPluginCreatorV3One() = default;
    virtual ~IPluginCreatorV3One() = default;
};

class ILogger : public IVersionedInterface
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"ILogger", 1, 0};
    }
    enum class Severity : int32_t
    {
        kINTERNAL_ERROR = 0,
        kERROR = 1,
        kWARNING = 2,
        kINFO = 3,
        kVERBOSE = 4
    };
    virtual void log(Severity severity, AsciiChar const* msg) noexcept = 0;
    ILogger() = default;
    ~ILogger() override = default;
};

class ILoggerFinder : public IVersionedInterface
{
public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"ILoggerFinder", 1, 0};
    }
    virtual ILogger* findLogger() = 0;

protected:
    ~ILoggerFinder() override = default;
};

class IPluginRegistry
{
public:
    using PluginLibraryHandle = void*;
    IPluginRegistry() = default;
    IPluginRegistry(IPluginRegistry const&) = delete;
    IPluginRegistry& operator=(IPluginRegistry const&) & = delete;

protected:
    virtual ~IPluginRegistry() noexcept = 0;

public:
    virtual void setErrorRecorder(IErrorRecorder* const recorder) noexcept = 0;
    virtual IErrorRecorder* getErrorRecorder() const noexcept = 0;
    virtual bool isParentSearchEnabled() const = 0;
    virtual void setParentSearchEnabled(bool const enabled) = 0;
    virtual PluginLibraryHandle loadLibrary(AsciiChar const* pluginPath) noexcept = 0;
    virtual void deregisterLibrary(PluginLibraryHandle handle) noexcept = 0;
    virtual bool registerCreator(IPluginCreatorInterface& creator, AsciiChar const* const pluginNamespace) noexcept = 0;
    virtual IPluginCreatorInterface* const* getAllCreators(int32_t* const numCreators) const noexcept = 0;
    virtual IPluginCreatorInterface* getCreator(AsciiChar const* const pluginName, AsciiChar const* const pluginVersion,
        AsciiChar const* const pluginNamespace = "") noexcept = 0;
    virtual bool deregisterCreator(IPluginCreatorInterface const& creator) noexcept = 0;
    virtual IPluginResource* acquirePluginResource(AsciiChar const* key, IPluginResource* resource) noexcept = 0;
    virtual int32_t releasePluginResource(AsciiChar const* key) noexcept = 0;
    virtual IPluginCreatorInterface* const* getAllCreatorsRecursive(int32_t* const numCreators) noexcept = 0;
};
inline IPluginRegistry::~IPluginRegistry() noexcept = default;

} // namespace nvinfer1

extern "C" TENSORRTAPI nvinfer1::IPluginRegistry* getPluginRegistry() noexcept;
extern "C" TENSORRTAPI nvinfer1::ILogger* getLogger() noexcept;
/* include/NvInferPlugin.h:29-40, plugin/api/inferPlugin.cpp:171-209 */
extern "C" TENSORRTAPI bool initLibNvInferPlugins(void* logger, char const* libNamespace);
/* plugin/vc/vfcCommon.cpp:68-79: the two symbols IPluginRegistry::loadLibrary looks up */
extern "C" TENSORRTAPI void setLoggerFinder(nvinfer1::ILoggerFinder* finder);
extern "C" TENSORRTAPI nvinfer1::IPluginCreatorInterface* const* getCreators(int32_t& nbCreators);

namespace nvinfer1
{
template <typename T>
class PluginRegistrar
{
public:
    PluginRegistrar()
    {
        getPluginRegistry()->registerCreator(instance, "");
    }

private:
    T instance{};
};
} // namespace nvinfer1

/* ---- the deprecated IPluginV2 family, kept because the reference still ships "Legacy" versions of the
 *      three BERT plugins on it (the *Legacy.h / *Legacy.cpp files of the three plugin directories) ------ */
struct cudnnContext;  /* never dereferenced: attachToContext() receives null on this platform */
struct cublasContext;

namespace nvinfer1
{
using PluginFormat = TensorFormat;

constexpr uint8_t kPLUGIN_VERSION_PYTHON_BIT = 0x40;
enum class PluginVersion : uint8_t
{
    kV2 = 0,
    kV2_EXT = 1,
    kV2_IOEXT = 2,
    kV2_DYNAMICEXT = 3,
    kV2_DYNAMICEXT_PYTHON = kPLUGIN_VERSION_PYTHON_BIT | 3
};

class IPluginV2
{
public:
    virtual int32_t getTensorRTVersion() const noexcept
    {
        return NV_TENSORRT_VERSION;
    }
    virtual AsciiChar const* getPluginType() const noexcept = 0;
    virtual AsciiChar const* getPluginVersion() const noexcept = 0;
    virtual int32_t getNbOutputs() const noexcept = 0;
    virtual Dims getOutputDimensions(int32_t index, Dims const* inputs, int32_t nbInputDims) noexcept = 0;
    virtual bool supportsFormat(DataType type, PluginFormat format) const noexcept = 0;
    virtual void configureWithFormat(Dims const* inputDims, int32_t nbInputs, Dims const* outputDims,
        int32_t nbOutputs, DataType type, PluginFormat format, int32_t maxBatchSize) noexcept = 0;
    virtual int32_t initialize() noexcept = 0;
    virtual void terminate() noexcept = 0;
    virtual size_t getWorkspaceSize(int32_t maxBatchSize) const noexcept = 0;
    virtual int32_t enqueue(int32_t batchSize, void const* const* inputs, void* const* outputs, void* workspace,
        hipStream_t stream) noexcept = 0;
    virtual size_t getSerializationSize() const noexcept = 0;
    virtual void serialize(void* buffer) const noexcept = 0;
    virtual void destroy() noexcept = 0;
    virtual IPluginV2* clone() const noexcept = 0;
    virtual void setPluginNamespace(AsciiChar const* pluginNamespace) noexcept = 0;
    virtual AsciiChar const* getPluginNamespace() const noexcept = 0;

    IPluginV2() = default;
    virtual ~IPluginV2() noexcept = default;

protected:
    IPluginV2(IPluginV2 const&) = default;
    IPluginV2(IPluginV2&&) = default;
    IPluginV2& operator=(IPluginV2 const&) & = default;
    IPluginV2& operator=(IPluginV2&&) & = default;
};

class IPluginV2Ext : public IPluginV2
{
public:
    virtual DataType getOutputDataType(int32_t index, DataType const* inputTypes, int32_t nbInputs) const noexcept = 0;
    virtual void configurePlugin(Dims const* inputDims, int32_t nbInputs, Dims const* outputDims, int32_t nbOutputs,
        DataType const* inputTypes, DataType const* outputTypes, bool const* inputIsBroadcast,
        bool const* outputIsBroadcast, PluginFormat floatFormat, int32_t maxBatchSize) noexcept = 0;

    IPluginV2Ext() = default;
    ~IPluginV2Ext() override = default;

    virtual void attachToContext(cudnnContext*, cublasContext*, IGpuAllocator*) noexcept {}
    virtual void detachFromContext() noexcept {}
    IPluginV2Ext* clone() const noexcept override = 0;

protected:
    IPluginV2Ext(IPluginV2Ext const&) = default;
    IPluginV2Ext(IPluginV2Ext&&) = default;
    IPluginV2Ext& operator=(IPluginV2Ext const&) & = default;
    IPluginV2Ext& operator=(IPluginV2Ext&&) & = default;

    int32_t getTensorRTVersion() const noexcept override
    {
        return static_cast<int32_t>((static_cast<uint32_t>(PluginVersion::kV2_EXT) << 24U)
            | (static_cast<uint32_t>(NV_TENSORRT_VERSION) & 0xFFFFFFU));
    }
    void configureWithFormat(Dims const*, int32_t, Dims const*, int32_t, DataType, PluginFormat, int32_t) noexcept override
    {
    }
};

class IPluginV2DynamicExt : public IPluginV2Ext
{
public:
    IPluginV2DynamicExt* clone() const noexcept override = 0;
    virtual DimsExprs getOutputDimensions(
        int32_t outputIndex, DimsExprs const* inputs, int32_t nbInputs, IExprBuilder& exprBuilder) noexcept = 0;
    static constexpr int32_t kFORMAT_COMBINATION_LIMIT = 100;
    virtual bool supportsFormatCombination(
        int32_t pos, PluginTensorDesc const* inOut, int32_t nbInputs, int32_t nbOutputs) noexcept = 0;
    virtual void configurePlugin(DynamicPluginTensorDesc const* in, int32_t nbInputs,
        DynamicPluginTensorDesc const* out, int32_t nbOutputs) noexcept = 0;
    virtual size_t getWorkspaceSize(PluginTensorDesc const* inputs, int32_t nbInputs, PluginTensorDesc const* outputs,
        int32_t nbOutputs) const noexcept = 0;
    virtual int32_t enqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc,
        void const* const* inputs, void* const* outputs, void* workspace, hipStream_t stream) noexcept = 0;

protected:
    int32_t getTensorRTVersion() const noexcept override
    {
        return (static_cast<int32_t>(PluginVersion::kV2_DYNAMICEXT) << 24 | (NV_TENSORRT_VERSION & 0xFFFFFF));
    }
    virtual ~IPluginV2DynamicExt() noexcept {}

private:
    /* the static-shape methods of the bases are closed off, as in the reference */
    void configurePlugin(Dims const*, int32_t, Dims const*, int32_t, DataType const*, DataType const*, bool const*,
        bool const*, PluginFormat, int32_t) noexcept final
    {
    }
    bool supportsFormat(DataType, PluginFormat) const noexcept final
    {
        return false;
    }
    Dims getOutputDimensions(int32_t, Dims const*, int32_t) noexcept final
    {
        return Dims{-1, {}};
    }
    size_t getWorkspaceSize(int32_t) const noexcept final
    {
        return 0;
    }
    int32_t enqueue(int32_t, void const* const*, void* const*, void*, hipStream_t) noexcept final
    {
        return 1;
    }
};

class IPluginCreator : public IPluginCreatorInterface
{
public:
    virtual AsciiChar const* getPluginName() const noexcept = 0;
    virtual AsciiChar const* getPluginVersion() const noexcept = 0;
    virtual PluginFieldCollection const* getFieldNames() noexcept = 0;
    virtual IPluginV2* createPlugin(AsciiChar const* name, PluginFieldCollection const* fc) noexcept = 0;
    virtual IPluginV2* deserializePlugin(AsciiChar const* name, void const* serialData, size_t serialLength) noexcept = 0;
    virtual void setPluginNamespace(AsciiChar const* pluginNamespace) noexcept = 0;
    virtual AsciiChar const* getPluginNamespace() const noexcept = 0;

    IPluginCreator() = default;
    ~IPluginCreator() override = default;

protected:
    IPluginCreator(IPluginCreator const&) = default;
    IPluginCreator(IPluginCreator&&) = default;
    IPluginCreator& operator=(IPluginCreator const&) & = default;
    IPluginCreator& operator=(IPluginCreator&&) & = default;

public:
    InterfaceInfo getInterfaceInfo() const noexcept override
    {
        return InterfaceInfo{"PLUGIN CREATOR_V1", 1, 0};
    }
};
} // namespace nvinfer1

#define REGISTER_TENSORRT_PLUGIN(name) static nvinfer1::PluginRegistrar<name> pluginRegistrar##name {}

#endif /* TRTAMD_NVINFER_API_H */
