// The "Legacy" versions of the three BERT plugins: the same operators on the deprecated
// IPluginV2DynamicExt / IPluginCreator interfaces, under the versions the reference registers them with
//   CustomEmbLayerNormPluginDynamic   1 (fixed length), 2 / 3 (var-seqlen HFace / MTron)
//       plugin/embLayerNormPlugin/embLayerNormPluginLegacy.cpp, embLayerNormVarSeqlenPluginLegacy.cpp:36-37
//   CustomSkipLayerNormPluginDynamic  1, 2 (var-seqlen), 3 / 4 (INT8 interleaved HFace / MTron)
//       plugin/skipLayerNormPlugin/skipLayerNormPluginLegacy.cpp:38-40, skipLayerNormInt8InterleavedPluginLegacy.cpp:35-36
//   CustomQKVToContextPluginDynamic   1, 2 (var-seqlen), 3 (INT8 interleaved)
//       plugin/bertQKVToContextPlugin/qkvToContextPluginLegacy.cpp:46-47, qkvToContextInt8InterleavedPluginLegacy.cpp:41
//
// The reference keeps two full implementations of every plugin.  Here a legacy plugin is an adapter
// around the IPluginV3 object of the matching current version (6/4/5, 5/6/7/8, 4/5/6): every V2 method
// maps onto one V3 method, and the serialised byte stream is the V3 plugin's serialised field list
// written out field by field, which deserializePlugin() turns back into a runtime-phase plugin.  The
// stream layout is this library's own (the reference's is a raw dump of its members, equally private
// to the library that wrote it).
#include "plugin_base.h"

#include <cstring>
#include <memory>
#include <string>
#include <vector>

namespace trtamd
{
namespace plugin
{
namespace
{

constexpr uint32_t kStreamMagic = 0x32564C50; // "PLV2"

size_t fieldElementSize(PluginFieldType t)
{
    switch (t)
    {
    case PluginFieldType::kFLOAT16: return 2;
    case PluginFieldType::kFLOAT32: return 4;
    case PluginFieldType::kFLOAT64: return 8;
    case PluginFieldType::kINT8: return 1;
    case PluginFieldType::kINT16: return 2;
    case PluginFieldType::kINT32: return 4;
    case PluginFieldType::kCHAR: return 1;
    case PluginFieldType::kDIMS: return sizeof(Dims);
    case PluginFieldType::kBF16: return 2;
    case PluginFieldType::kINT64: return 8;
    case PluginFieldType::kFP8: return 1;
    case PluginFieldType::kINT4: return 1;
    case PluginFieldType::kFP4: return 1;
    case PluginFieldType::kUNKNOWN: return 1; // raw bytes (the attention plugins' runner state)
    default: return 0;
    }
}

size_t pad8(size_t n)
{
    return (n + 7) & ~size_t(7);
}

// [magic u32][nbFields u32] then per field [nameLen u32][type i32][length i32][pad u32][name, padded to 8]
// [data, padded to 8]
size_t streamSize(PluginFieldCollection const& fc)
{
    size_t n = 8;
    for (int32_t i = 0; i < fc.nbFields; ++i)
    {
        PluginField const& f = fc.fields[i];
        n += 16 + pad8(std::strlen(f.name)) + pad8(fieldElementSize(f.type) * static_cast<size_t>(f.length));
    }
    return n;
}

void writeStream(PluginFieldCollection const& fc, uint8_t* out)
{
    auto put32 = [&](uint32_t v) {
        std::memcpy(out, &v, 4);
        out += 4;
    };
    put32(kStreamMagic);
    put32(static_cast<uint32_t>(fc.nbFields));
    for (int32_t i = 0; i < fc.nbFields; ++i)
    {
        PluginField const& f = fc.fields[i];
        size_t const nameLen = std::strlen(f.name);
        size_t const bytes = fieldElementSize(f.type) * static_cast<size_t>(f.length);
        put32(static_cast<uint32_t>(nameLen));
        put32(static_cast<uint32_t>(f.type));
        put32(static_cast<uint32_t>(f.length));
        put32(0);
        std::memset(out, 0, pad8(nameLen));
        std::memcpy(out, f.name, nameLen);
        out += pad8(nameLen);
        std::memset(out, 0, pad8(bytes));
        if (bytes)
        {
            std::memcpy(out, f.data, bytes);
        }
        out += pad8(bytes);
    }
}

// Parsed stream: owns the names; data pointers refer into the caller's buffer (8-byte aligned offsets).
struct ParsedStream
{
    std::vector<std::string> names;
    std::vector<PluginField> fields;
    PluginFieldCollection fc{};
};

void parseStream(void const* data, size_t length, ParsedStream& ps)
{
    auto const* p = static_cast<uint8_t const*>(data);
    auto const* end = p + length;
    auto need = [&](size_t n) {
        if (static_cast<size_t>(end - p) < n)
        {
            throw std::runtime_error("serialised plugin is truncated");
        }
    };
    auto get32 = [&]() {
        need(4);
        uint32_t v;
        std::memcpy(&v, p, 4);
        p += 4;
        return v;
    };
    if (data == nullptr || get32() != kStreamMagic)
    {
        throw std::runtime_error("not a plugin stream written by this library");
    }
    uint32_t const n = get32();
    if (static_cast<size_t>(n) > length / 16)
    {
        throw std::runtime_error("serialised plugin is truncated"); // every field takes at least its 16-byte header
    }
    ps.names.reserve(n);
    for (uint32_t i = 0; i < n; ++i)
    {
        uint32_t const nameLen = get32();
        auto const type = static_cast<PluginFieldType>(get32());
        auto const len = static_cast<int32_t>(get32());
        get32();
        need(pad8(nameLen));
        ps.names.emplace_back(reinterpret_cast<char const*>(p), nameLen);
        p += pad8(nameLen);
        size_t const bytes = fieldElementSize(type) * static_cast<size_t>(len < 0 ? 0 : len);
        need(pad8(bytes));
        ps.fields.emplace_back(nullptr, bytes ? p : nullptr, type, len);
        p += pad8(bytes);
    }
    for (size_t i = 0; i < ps.fields.size(); ++i)
    {
        ps.fields[i].name = ps.names[i].c_str();
    }
    ps.fc.nbFields = static_cast<int32_t>(ps.fields.size());
    ps.fc.fields = ps.fields.data();
}

struct V3Deleter
{
    void operator()(IPluginV3* p) const
    {
        delete p;
    }
};
using V3Ptr = std::unique_ptr<IPluginV3, V3Deleter>;

template <typename T>
T* cap(IPluginV3* p, PluginCapabilityType t)
{
    return static_cast<T*>(p->getCapabilityInterface(t));
}

std::vector<DynamicPluginTensorDesc> widen(PluginTensorDesc const* d, int32_t n)
{
    std::vector<DynamicPluginTensorDesc> v(static_cast<size_t>(n > 0 ? n : 0));
    for (int32_t i = 0; i < n; ++i)
    {
        v[i].desc = d[i];
        v[i].min = v[i].max = v[i].opt = d[i].dims;
    }
    return v;
}

class LegacyAdapter final : public IPluginV2DynamicExt
{
public:
    LegacyAdapter(V3Ptr plugin, char const* legacyVersion, std::string ns, int32_t nbInputs)
        : mPlugin(std::move(plugin))
        , mVersion(legacyVersion)
        , mNamespace(std::move(ns))
        , mNbInputs(nbInputs)
    {
        mCore = cap<IPluginV3OneCore>(mPlugin.get(), PluginCapabilityType::kCORE);
        mBuild = cap<IPluginV3OneBuild>(mPlugin.get(), PluginCapabilityType::kBUILD);
        mRuntime = cap<IPluginV3OneRuntime>(mPlugin.get(), PluginCapabilityType::kRUNTIME);
    }

    // IPluginV2
    AsciiChar const* getPluginType() const noexcept override
    {
        return mCore->getPluginName();
    }
    AsciiChar const* getPluginVersion() const noexcept override
    {
        return mVersion;
    }
    int32_t getNbOutputs() const noexcept override
    {
        return mBuild->getNbOutputs();
    }
    int32_t initialize() noexcept override
    {
        return 0;
    }
    void terminate() noexcept override {}
    size_t getSerializationSize() const noexcept override
    {
        PluginFieldCollection const* fc = mRuntime->getFieldsToSerialize();
        return fc ? streamSize(*fc) : 0;
    }
    void serialize(void* buffer) const noexcept override
    {
        PluginFieldCollection const* fc = mRuntime->getFieldsToSerialize();
        if (fc && buffer)
        {
            writeStream(*fc, static_cast<uint8_t*>(buffer));
        }
    }
    void destroy() noexcept override
    {
        delete this;
    }
    void setPluginNamespace(AsciiChar const* pluginNamespace) noexcept override
    {
        try
        {
            mNamespace = pluginNamespace ? pluginNamespace : "";
        }
        catch (...)
        {
        }
    }
    AsciiChar const* getPluginNamespace() const noexcept override
    {
        return mNamespace.c_str();
    }

    // IPluginV2Ext
    DataType getOutputDataType(int32_t index, DataType const* inputTypes, int32_t nbInputs) const noexcept override
    {
        int32_t const nb = mBuild->getNbOutputs();
        DataType types[8] = {};
        if (index < 0 || index >= nb || nb > 8 || mBuild->getOutputDataTypes(types, nb, inputTypes, nbInputs) != 0)
        {
            return DataType::kFLOAT;
        }
        return types[index];
    }

    // IPluginV2DynamicExt
    IPluginV2DynamicExt* clone() const noexcept override
    {
        try
        {
            V3Ptr copy(mPlugin->clone());
            if (!copy)
            {
                return nullptr;
            }
            return new LegacyAdapter(std::move(copy), mVersion, mNamespace, mNbInputs);
        }
        catch (...)
        {
            return nullptr;
        }
    }
    DimsExprs getOutputDimensions(
        int32_t outputIndex, DimsExprs const* inputs, int32_t nbInputs, IExprBuilder& exprBuilder) noexcept override
    {
        DimsExprs outs[8] = {};
        int32_t const nb = mBuild->getNbOutputs();
        DimsExprs bad{};
        bad.nbDims = -1;
        if (outputIndex < 0 || outputIndex >= nb || nb > 8
            || mBuild->getOutputShapes(inputs, nbInputs, nullptr, 0, outs, nb, exprBuilder) != 0)
        {
            return bad;
        }
        return outs[outputIndex];
    }
    bool supportsFormatCombination(
        int32_t pos, PluginTensorDesc const* inOut, int32_t nbInputs, int32_t nbOutputs) noexcept override
    {
        try
        {
            mNbInputs = nbInputs;
            auto v = widen(inOut, nbInputs + nbOutputs);
            return mBuild->supportsFormatCombination(pos, v.data(), nbInputs, nbOutputs);
        }
        catch (...)
        {
            return false;
        }
    }
    void configurePlugin(DynamicPluginTensorDesc const* in, int32_t nbInputs, DynamicPluginTensorDesc const* out,
        int32_t nbOutputs) noexcept override
    {
        mNbInputs = nbInputs;
        mBuild->configurePlugin(in, nbInputs, out, nbOutputs);
    }
    size_t getWorkspaceSize(PluginTensorDesc const* inputs, int32_t nbInputs, PluginTensorDesc const* outputs,
        int32_t nbOutputs) const noexcept override
    {
        try
        {
            auto i = widen(inputs, nbInputs);
            auto o = widen(outputs, nbOutputs);
            return mBuild->getWorkspaceSize(i.data(), nbInputs, o.data(), nbOutputs);
        }
        catch (...)
        {
            return 0;
        }
    }
    int32_t enqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void* workspace, hipStream_t stream) noexcept override
    {
        // a V2 plugin learns its shapes in enqueue(); the V3 object wants them through onShapeChange() first.
        // The V2 signature carries no input count: it is the one the plugin was created or configured with.
        int32_t const st = mRuntime->onShapeChange(inputDesc, mNbInputs, outputDesc, mBuild->getNbOutputs());
        if (st != 0)
        {
            return st;
        }
        return mRuntime->enqueue(inputDesc, outputDesc, inputs, outputs, workspace, stream);
    }

private:
    V3Ptr mPlugin;
    IPluginV3OneCore* mCore{};
    IPluginV3OneBuild* mBuild{};
    IPluginV3OneRuntime* mRuntime{};
    char const* mVersion;
    std::string mNamespace;
    int32_t mNbInputs;
};

// How many inputs each operator takes, from its serialised configuration (needed because the V2
// enqueue() does not say): SkipLayerNorm 2; EmbLayerNorm fixed 3, var-seqlen 4; QKV-to-context 1 + has_mask
// + 2 * var_seqlen, interleaved 3.
int32_t inputsOf(char const* pluginName, char const* legacyVersion, IPluginV3* p)
{
    std::string const name = pluginName;
    int const v = std::atoi(legacyVersion);
    if (name == "CustomSkipLayerNormPluginDynamic")
    {
        return 2;
    }
    if (name == "CustomEmbLayerNormPluginDynamic")
    {
        return v == 1 ? 3 : 4;
    }
    if (v == 3)
    {
        return 3;
    }
    PluginFieldCollection const* fc = cap<IPluginV3OneRuntime>(p, PluginCapabilityType::kRUNTIME)->getFieldsToSerialize();
    auto flag = [&](char const* field, int32_t fallback) {
        for (int32_t i = 0; fc && i < fc->nbFields; ++i)
        {
            if (std::strcmp(fc->fields[i].name, field) == 0 && fc->fields[i].data
                && fc->fields[i].type == PluginFieldType::kINT32 && fc->fields[i].length >= 1)
            {
                return *static_cast<int32_t const*>(fc->fields[i].data);
            }
        }
        return fallback;
    };
    // qkv, the mask when has_mask was set, and for version 2 cu_seqlens and the max-length dummy when var_seqlen is
    // set (plugin/bertQKVToContextPlugin/qkvToContextPluginLegacy.cpp, QKVToContextVarSeqlenPluginDynamicLegacy)
    int32_t const varSeqlen = v == 2 && flag("var_seqlen", 0) != 0 ? 1 : 0;
    return 1 + (flag("has_mask", 1) != 0 ? 1 : 0) + 2 * varSeqlen;
}

class LegacyCreator : public IPluginCreator
{
public:
    LegacyCreator(char const* name, char const* legacyVersion, char const* currentVersion)
        : mName(name)
        , mVersion(legacyVersion)
        , mCurrent(currentVersion)
    {
        recordCreator(this);
    }

    AsciiChar const* getPluginName() const noexcept override
    {
        return mName;
    }
    AsciiChar const* getPluginVersion() const noexcept override
    {
        return mVersion;
    }
    PluginFieldCollection const* getFieldNames() noexcept override
    {
        auto* c = current();
        return c ? c->getFieldNames() : nullptr;
    }
    IPluginV2* createPlugin(AsciiChar const* name, PluginFieldCollection const* fc) noexcept override
    {
        return make(name, fc, TensorRTPhase::kBUILD);
    }
    IPluginV2* deserializePlugin(AsciiChar const* name, void const* serialData, size_t serialLength) noexcept override
    {
        try
        {
            ParsedStream ps;
            parseStream(serialData, serialLength, ps);
            return make(name, &ps.fc, TensorRTPhase::kRUNTIME);
        }
        catch (std::exception const& e)
        {
            logError(e.what());
        }
        catch (...)
        {
            logError("unknown error while reading the serialised plugin");
        }
        return nullptr;
    }
    void setPluginNamespace(AsciiChar const* pluginNamespace) noexcept override
    {
        try
        {
            mNamespace = pluginNamespace ? pluginNamespace : "";
        }
        catch (...)
        {
        }
    }
    AsciiChar const* getPluginNamespace() const noexcept override
    {
        return mNamespace.c_str();
    }

private:
    IPluginCreatorV3One* current()
    {
        return static_cast<IPluginCreatorV3One*>(getPluginRegistry()->getCreator(mName, mCurrent, ""));
    }
    IPluginV2* make(AsciiChar const* name, PluginFieldCollection const* fc, TensorRTPhase phase) noexcept
    {
        try
        {
            auto* c = current();
            if (!c)
            {
                logError("the current-version creator of this plugin is not registered");
                return nullptr;
            }
            V3Ptr p(c->createPlugin(name ? name : "", fc, phase));
            if (!p)
            {
                return nullptr; // the V3 creator has logged why
            }
            int32_t const nbIn = inputsOf(mName, mVersion, p.get());
            return new LegacyAdapter(std::move(p), mVersion, mNamespace, nbIn);
        }
        catch (std::exception const& e)
        {
            logError(e.what());
        }
        return nullptr;
    }
    void logError(char const* what) noexcept
    {
        if (ILogger* l = getLogger())
        {
            std::string msg = std::string(mName) + " version " + mVersion + ": " + what;
            l->log(ILogger::Severity::kERROR, msg.c_str());
        }
    }

    char const* mName;
    char const* mVersion;
    char const* mCurrent;
    std::string mNamespace;
};

#define TRTAMD_LEGACY_CREATOR(cls, name, legacy, current)                                                              \
    class cls final : public LegacyCreator                                                                             \
    {                                                                                                                  \
    public:                                                                                                            \
        cls()                                                                                                          \
            : LegacyCreator(name, legacy, current)                                                                     \
        {                                                                                                              \
        }                                                                                                              \
    };                                                                                                                 \
    REGISTER_TENSORRT_PLUGIN(cls)

TRTAMD_LEGACY_CREATOR(EmbLayerNormLegacyCreator, "CustomEmbLayerNormPluginDynamic", "1", "6");
TRTAMD_LEGACY_CREATOR(EmbLayerNormVarSeqlenHFaceLegacyCreator, "CustomEmbLayerNormPluginDynamic", "2", "4");
TRTAMD_LEGACY_CREATOR(EmbLayerNormVarSeqlenMTronLegacyCreator, "CustomEmbLayerNormPluginDynamic", "3", "5");
TRTAMD_LEGACY_CREATOR(SkipLayerNormLegacyCreator, "CustomSkipLayerNormPluginDynamic", "1", "5");
TRTAMD_LEGACY_CREATOR(SkipLayerNormVarSeqlenLegacyCreator, "CustomSkipLayerNormPluginDynamic", "2", "6");
TRTAMD_LEGACY_CREATOR(SkipLayerNormInterleavedHFaceLegacyCreator, "CustomSkipLayerNormPluginDynamic", "3", "7");
TRTAMD_LEGACY_CREATOR(SkipLayerNormInterleavedMTronLegacyCreator, "CustomSkipLayerNormPluginDynamic", "4", "8");
TRTAMD_LEGACY_CREATOR(QkvToContextLegacyCreator, "CustomQKVToContextPluginDynamic", "1", "4");
TRTAMD_LEGACY_CREATOR(QkvToContextVarSeqlenLegacyCreator, "CustomQKVToContextPluginDynamic", "2", "5");
TRTAMD_LEGACY_CREATOR(QkvToContextInterleavedLegacyCreator, "CustomQKVToContextPluginDynamic", "3", "6");

} // namespace
} // namespace plugin
} // namespace trtamd
