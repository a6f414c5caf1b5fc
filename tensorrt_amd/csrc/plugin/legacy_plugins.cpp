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
// maps onto one V3 method.  serialize() writes the byte layout of the reference's legacy classes (their
// members in the order and widths of their serialize() functions: bool 1 byte, int32_t / DataType / float 4,
// size_t 8, weights as raw arrays, no padding; plugin/common/serialize.hpp:43-65, bertCommon.h:219-225), built
// from the V3 plugin's serialised field list; deserializePlugin() reads that layout back into the field list
// that creates the runtime-phase V3 plugin.
//   embLayerNormPluginLegacy.cpp (serialize), embLayerNormVarSeqlenPluginLegacy.cpp:544-562,
//   skipLayerNormPluginLegacy.cpp:381-402, skipLayerNormInt8InterleavedPluginLegacy.cpp (serialize),
//   qkvToContextPluginLegacy.cpp:399-422, 909-925, qkvToContextInt8InterleavedPluginLegacy.cpp (serialize),
//   runner state: mhaRunner.cu:456-507.
#include "plugin_base.h"

#include <cstring>
#include <deque>
#include <memory>
#include <string>
#include <vector>

namespace trtamd
{
namespace plugin
{
namespace
{

enum class Layout
{
    kEMB_FIXED,        // CustomEmbLayerNormPluginDynamic 1
    kEMB_VARSEQLEN,    // 2 (HFace), 3 (MTron)
    kSKIP,             // CustomSkipLayerNormPluginDynamic 1, 2
    kSKIP_INTERLEAVED, // 3, 4
    kQKV,              // CustomQKVToContextPluginDynamic 1
    kQKV_VARSEQLEN,    // 2
    kQKV_INTERLEAVED,  // 3
};

// What the legacy classes keep as members that the V3 field lists do not carry.
struct Extras
{
    int64_t S{0};   // EmbLayerNorm 1: the sequence length seen by configurePlugin
    bool mtron{false};
};

class ByteWriter
{
public:
    template <typename T>
    void put(T v)
    {
        auto const* p = reinterpret_cast<uint8_t const*>(&v);
        mBuf.insert(mBuf.end(), p, p + sizeof(T));
    }
    void bytes(void const* p, size_t n)
    {
        auto const* b = static_cast<uint8_t const*>(p);
        mBuf.insert(mBuf.end(), b, b + n);
    }
    std::vector<uint8_t> const& data() const
    {
        return mBuf;
    }

private:
    std::vector<uint8_t> mBuf;
};

class ByteReader
{
public:
    ByteReader(void const* data, size_t length)
        : mP(static_cast<uint8_t const*>(data))
        , mEnd(mP + (data ? length : 0))
    {
        if (data == nullptr)
        {
            throw std::runtime_error("serialised plugin is truncated");
        }
    }
    template <typename T>
    T get()
    {
        T v;
        std::memcpy(&v, span(sizeof(T)), sizeof(T));
        return v;
    }
    bool flag()
    {
        return get<uint8_t>() != 0;
    }
    uint8_t const* span(size_t n)
    {
        if (static_cast<size_t>(mEnd - mP) < n)
        {
            throw std::runtime_error("serialised plugin is truncated");
        }
        uint8_t const* p = mP;
        mP += n;
        return p;
    }
    // element counts come from the stream: refuse what cannot fit before multiplying
    size_t count(uint64_t n, size_t elemBytes)
    {
        if (n > static_cast<uint64_t>(mEnd - mP) / (elemBytes ? elemBytes : 1))
        {
            throw std::runtime_error("serialised plugin is truncated");
        }
        return static_cast<size_t>(n);
    }

private:
    uint8_t const* mP;
    uint8_t const* mEnd;
};

// The field list handed to createPlugin(kRUNTIME): owns its values (8-byte aligned copies, because nothing in the
// reference's byte layout is aligned).
class FieldStore
{
public:
    void i32(char const* name, int32_t v)
    {
        raw(name, &v, 4, PluginFieldType::kINT32, 1);
    }
    void f32(char const* name, float v)
    {
        raw(name, &v, 4, PluginFieldType::kFLOAT32, 1);
    }
    void raw(char const* name, void const* p, size_t bytes, PluginFieldType type, int32_t length)
    {
        mBlobs.emplace_back((bytes + 7) / 8 + 1);
        std::memcpy(mBlobs.back().data(), p, bytes);
        mFields.emplace_back(name, mBlobs.back().data(), type, length);
    }
    PluginFieldCollection collection()
    {
        return PluginFieldCollection{static_cast<int32_t>(mFields.size()), mFields.data()};
    }

private:
    std::deque<std::vector<uint64_t>> mBlobs;
    std::vector<PluginField> mFields;
};

PluginField const* fieldOf(PluginFieldCollection const& fc, char const* name)
{
    for (int32_t i = 0; i < fc.nbFields; ++i)
    {
        if (fc.fields[i].name && std::strcmp(fc.fields[i].name, name) == 0 && fc.fields[i].data)
        {
            return &fc.fields[i];
        }
    }
    return nullptr;
}

int32_t i32Of(PluginFieldCollection const& fc, char const* name, int32_t fallback)
{
    PluginField const* f = fieldOf(fc, name);
    return f && f->type == PluginFieldType::kINT32 && f->length >= 1 ? *static_cast<int32_t const*>(f->data) : fallback;
}

float f32Of(PluginFieldCollection const& fc, char const* name, float fallback)
{
    PluginField const* f = fieldOf(fc, name);
    return f && f->type == PluginFieldType::kFLOAT32 && f->length >= 1 ? *static_cast<float const*>(f->data) : fallback;
}

size_t weightBytes(PluginField const& f)
{
    return static_cast<size_t>(f.length) * (f.type == PluginFieldType::kFLOAT16 ? 2 : 4);
}

PluginField const& required(PluginFieldCollection const& fc, char const* name)
{
    PluginField const* f = fieldOf(fc, name);
    if (!f)
    {
        throw std::runtime_error(std::string("the plugin does not serialise its field ") + name);
    }
    return *f;
}

constexpr char const* kEMB_BETA = "bert_embeddings_layernorm_beta";
constexpr char const* kEMB_GAMMA = "bert_embeddings_layernorm_gamma";
constexpr char const* kEMB_WORD = "bert_embeddings_word_embeddings";
constexpr char const* kEMB_TOK = "bert_embeddings_token_type_embeddings";
constexpr char const* kEMB_POS = "bert_embeddings_position_embeddings";

// ---- V3 field list -> the legacy class's bytes ---------------------------------------------------------------
std::vector<uint8_t> encode(Layout layout, PluginFieldCollection const& fc, Extras const& ex)
{
    ByteWriter w;
    auto const half = static_cast<int32_t>(DataType::kHALF);
    auto const flt = static_cast<int32_t>(DataType::kFLOAT);
    switch (layout)
    {
    case Layout::kEMB_FIXED:
    case Layout::kEMB_VARSEQLEN:
    {
        PluginField const& beta = required(fc, kEMB_BETA);
        PluginField const& gamma = required(fc, kEMB_GAMMA);
        PluginField const& word = required(fc, kEMB_WORD);
        PluginField const& pos = required(fc, kEMB_POS);
        PluginField const& tok = required(fc, kEMB_TOK);
        int32_t const type = i32Of(fc, "output_fp16", 0) ? half : flt;
        uint64_t const ld = static_cast<uint64_t>(beta.length);
        uint64_t const wv = ld ? word.length / ld : 0, pv = ld ? pos.length / ld : 0, tv = ld ? tok.length / ld : 0;
        w.put<int32_t>(type);                                              // mType
        if (layout == Layout::kEMB_FIXED)
        {
            w.put<int32_t>(i32Of(fc, "mha_type_id", flt));                 // mMhaType
            w.put<uint64_t>(ld);                                           // mLd
            w.put<uint64_t>(static_cast<uint64_t>(ex.S));                  // mS
            w.put<uint64_t>(wv);                                           // mWordVocabSize
            w.put<uint64_t>(pv);                                           // mPosVocabSize
            w.put<uint64_t>(tv);                                           // mTokVocabSize
            w.put<uint8_t>(i32Of(fc, "full_mask", 0) != 0);                // mUseFullMask
            w.put<int32_t>(getSmVersion());                                // mSM
        }
        else
        {
            w.put<uint64_t>(ld);
            w.put<uint64_t>(wv);
            w.put<uint64_t>(pv);
            w.put<uint64_t>(tv);
            w.put<int32_t>(ex.mtron ? type : static_cast<int32_t>(DataType::kINT32)); // mMaskType
        }
        w.bytes(beta.data, weightBytes(beta));                             // binary32 [ld]
        w.bytes(gamma.data, weightBytes(gamma));
        w.bytes(word.data, weightBytes(word));                             // mType [vocab][ld]
        w.bytes(pos.data, weightBytes(pos));
        w.bytes(tok.data, weightBytes(tok));
        break;
    }
    case Layout::kSKIP:
    {
        PluginField const& beta = required(fc, "beta");
        PluginField const& gamma = required(fc, "gamma");
        PluginField const* bias = fieldOf(fc, "bias");
        int32_t const type = i32Of(fc, "type_id", flt);
        w.put<int32_t>(type);                                              // mType
        w.put<int32_t>(beta.type == PluginFieldType::kFLOAT16 ? half : flt); // mCfgType
        w.put<uint64_t>(static_cast<uint64_t>(beta.length));               // mLd
        w.put<uint8_t>(bias != nullptr);                                   // mHasBias
        w.bytes(beta.data, weightBytes(beta));
        w.bytes(gamma.data, weightBytes(gamma));
        if (bias)
        {
            w.bytes(bias->data, weightBytes(*bias));
        }
        break;
    }
    case Layout::kSKIP_INTERLEAVED:
    {
        PluginField const& beta = required(fc, "beta");
        PluginField const& gamma = required(fc, "gamma");
        w.put<uint64_t>(static_cast<uint64_t>(beta.length));               // mLd
        w.bytes(beta.data, weightBytes(beta));                             // binary16 [ld]
        w.bytes(gamma.data, weightBytes(gamma));
        break;
    }
    case Layout::kQKV:
    case Layout::kQKV_VARSEQLEN:
    {
        int32_t const hidden = i32Of(fc, "hidden_size", 0), heads = i32Of(fc, "num_heads", 0);
        w.put<int32_t>(i32Of(fc, "type_id", flt));                         // mType
        w.put<int32_t>(heads);                                             // mNumHeads
        w.put<int32_t>(heads > 0 ? hidden / heads : 0);                    // mHeadSize
        w.put<uint8_t>(i32Of(fc, "has_mask", 0) != 0);                     // mHasImask
        w.put<int32_t>(hidden);                                            // mHiddenSize
        w.put<int32_t>(i32Of(fc, "SM", getSmVersion()));                   // mSM
        w.put<int32_t>(i32Of(fc, "S", 0));                                 // mS
        w.put<int32_t>(i32Of(fc, "B", 0));                                 // mB
        w.put<float>(f32Of(fc, "dq_probs", -1.F));                         // mDqProbs
        PluginField const* runner = fieldOf(fc, "runnerStateBuffer");
        if (layout == Layout::kQKV)
        {
            bool const has = runner != nullptr && i32Of(fc, "hasUnfusedDispatcher", 0) != 0;
            w.put<int32_t>(has ? 1 : 0);                                   // hasUnfusedRunner
            if (has)
            {
                w.bytes(runner->data, static_cast<size_t>(runner->length)); // algo1, algo2, S, B, headSize
            }
        }
        else
        {
            bool const varSeqlen = i32Of(fc, "var_seqlen", 0) != 0;
            w.put<uint8_t>(varSeqlen);                                     // mUseVarSeqlen
            w.put<int32_t>(varSeqlen ? 1 : 2);                             // mHdim
            w.put<uint8_t>(i32Of(fc, "use_int8_scale_max", 1) != 0);       // mUseInt8ScaleMax
            if (!runner)
            {
                throw std::runtime_error("the attention plugin has no runner yet (configurePlugin first)");
            }
            w.bytes(runner->data, static_cast<size_t>(runner->length));    // S, B, headSize (after algo1, algo2 if unfused)
        }
        break;
    }
    case Layout::kQKV_INTERLEAVED:
    {
        int32_t const hidden = i32Of(fc, "hidden_size", 0), heads = i32Of(fc, "num_heads", 0);
        w.put<int32_t>(heads);                                             // mNumHeads
        w.put<int32_t>(heads > 0 ? hidden / heads : 0);                    // mHeadSize
        w.put<int32_t>(hidden);                                            // mHiddenSize
        w.put<int32_t>(getSmVersion());                                    // mSM
        w.put<int32_t>(0);                                                 // mS (never set by the reference either)
        w.put<int32_t>(0);                                                 // mB
        w.put<float>(f32Of(fc, "dq_probs", -1.F));                         // mDqProbs
        w.put<uint8_t>(i32Of(fc, "use_int8_scale_max", 1) != 0);           // mUseInt8ScaleMax
        w.put<uint8_t>(i32Of(fc, "use_explicit_int8", 0) != 0);            // mUseExplicitInt8
        w.put<float>(f32Of(fc, "input_qkv_scale", 0.F));                   // mQkvScale
        w.put<float>(f32Of(fc, "output_ctx_scale", 0.F));                  // mCtxScale
        break;
    }
    }
    return w.data();
}

// ---- the legacy class's bytes -> the field list of the runtime-phase V3 plugin --------------------------------
void decode(Layout layout, void const* data, size_t length, FieldStore& fs, Extras& ex)
{
    ByteReader r(data, length);
    auto const half = static_cast<int32_t>(DataType::kHALF);
    auto weights = [&](char const* name, uint64_t n, bool fp16) {
        size_t const eb = fp16 ? 2 : 4;
        size_t const cnt = r.count(n, eb);
        if (cnt > 0x7fffffffULL)
        {
            throw std::runtime_error("serialised plugin holds a weight array beyond 2^31 elements");
        }
        fs.raw(name, r.span(cnt * eb), cnt * eb, fp16 ? PluginFieldType::kFLOAT16 : PluginFieldType::kFLOAT32,
            static_cast<int32_t>(cnt));
    };
    switch (layout)
    {
    case Layout::kEMB_FIXED:
    case Layout::kEMB_VARSEQLEN:
    {
        int32_t const type = r.get<int32_t>();
        bool const fp16 = type == half;
        uint64_t ld, wv, pv, tv;
        if (layout == Layout::kEMB_FIXED)
        {
            fs.i32("mha_type_id", r.get<int32_t>());
            ld = r.get<uint64_t>();
            ex.S = static_cast<int64_t>(r.get<uint64_t>());
            wv = r.get<uint64_t>();
            pv = r.get<uint64_t>();
            tv = r.get<uint64_t>();
            fs.i32("full_mask", r.flag() ? 1 : 0);
            (void) r.get<int32_t>(); // mSM: the architecture the stream was written on
        }
        else
        {
            ld = r.get<uint64_t>();
            wv = r.get<uint64_t>();
            pv = r.get<uint64_t>();
            tv = r.get<uint64_t>();
            (void) r.get<int32_t>(); // mMaskType follows from the version
        }
        fs.i32("output_fp16", fp16 ? 1 : 0);
        size_t const n = r.count(ld, 4);
        weights(kEMB_BETA, n, false);
        weights(kEMB_GAMMA, n, false);
        size_t const eb = fp16 ? 2 : 4;
        weights(kEMB_WORD, static_cast<uint64_t>(n) * r.count(wv, n * eb ? n * eb : 1), fp16);
        weights(kEMB_POS, static_cast<uint64_t>(n) * r.count(pv, n * eb ? n * eb : 1), fp16);
        weights(kEMB_TOK, static_cast<uint64_t>(n) * r.count(tv, n * eb ? n * eb : 1), fp16);
        break;
    }
    case Layout::kSKIP:
    {
        fs.i32("type_id", r.get<int32_t>());
        bool const fp16 = r.get<int32_t>() == half;
        uint64_t const ld = r.get<uint64_t>();
        bool const hasBias = r.flag();
        if (ld > 0x7fffffffULL)
        {
            throw std::runtime_error("serialised plugin is truncated");
        }
        fs.i32("ld", static_cast<int32_t>(ld));
        weights("beta", ld, fp16);
        weights("gamma", ld, fp16);
        if (hasBias)
        {
            weights("bias", ld, fp16);
        }
        break;
    }
    case Layout::kSKIP_INTERLEAVED:
    {
        uint64_t const ld = r.get<uint64_t>();
        weights("beta", ld, true);
        weights("gamma", ld, true);
        break;
    }
    case Layout::kQKV:
    case Layout::kQKV_VARSEQLEN:
    {
        int32_t const type = r.get<int32_t>();
        fs.i32("type_id", type);
        fs.i32("num_heads", r.get<int32_t>());
        (void) r.get<int32_t>(); // mHeadSize = hidden / heads
        fs.i32("has_mask", r.flag() ? 1 : 0);
        fs.i32("hidden_size", r.get<int32_t>());
        int32_t const sm = r.get<int32_t>();
        fs.i32("S", r.get<int32_t>());
        fs.i32("B", r.get<int32_t>());
        float const dqProbs = r.get<float>();
        if (dqProbs >= 0.F)
        {
            fs.f32("dq_probs", dqProbs);
        }
        if (layout == Layout::kQKV)
        {
            fs.i32("SM", sm);
            int32_t const has = r.get<int32_t>();
            fs.i32("hasUnfusedDispatcher", has != 0 ? 1 : 0);
            if (has != 0)
            {
                fs.raw("runnerStateBuffer", r.span(20), 20, PluginFieldType::kUNKNOWN, 20);
            }
        }
        else
        {
            bool const varSeqlen = r.flag();
            fs.i32("var_seqlen", varSeqlen ? 1 : 0);
            (void) r.get<int32_t>(); // mHdim follows from var_seqlen
            fs.i32("use_int8_scale_max", r.flag() ? 1 : 0);
            size_t const n = varSeqlen ? 12 : 20; // fused runner: S, B, headSize; unfused: two algorithms first
            fs.raw("runnerStateBuffer", r.span(n), n, PluginFieldType::kUNKNOWN, static_cast<int32_t>(n));
        }
        break;
    }
    case Layout::kQKV_INTERLEAVED:
    {
        fs.i32("num_heads", r.get<int32_t>());
        (void) r.get<int32_t>();
        fs.i32("hidden_size", r.get<int32_t>());
        (void) r.get<int32_t>(); // mSM
        (void) r.get<int32_t>(); // mS
        (void) r.get<int32_t>(); // mB
        float const dqProbs = r.get<float>();
        if (dqProbs >= 0.F)
        {
            fs.f32("dq_probs", dqProbs);
        }
        fs.i32("use_int8_scale_max", r.flag() ? 1 : 0);
        fs.i32("use_explicit_int8", r.flag() ? 1 : 0);
        fs.f32("input_qkv_scale", r.get<float>());
        fs.f32("output_ctx_scale", r.get<float>());
        break;
    }
    }
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
    LegacyAdapter(V3Ptr plugin, char const* legacyVersion, std::string ns, int32_t nbInputs, Layout layout,
        Extras const& extras)
        : mPlugin(std::move(plugin))
        , mVersion(legacyVersion)
        , mNamespace(std::move(ns))
        , mNbInputs(nbInputs)
        , mLayout(layout)
        , mExtras(extras)
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
        return encoded().size();
    }
    void serialize(void* buffer) const noexcept override
    {
        std::vector<uint8_t> const bytes = encoded();
        if (buffer && !bytes.empty())
        {
            std::memcpy(buffer, bytes.data(), bytes.size());
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
            return new LegacyAdapter(std::move(copy), mVersion, mNamespace, mNbInputs, mLayout, mExtras);
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
        if (mLayout == Layout::kEMB_FIXED && in && nbInputs > 0 && in[0].desc.dims.nbDims > 0)
        {
            mExtras.S = in[0].desc.dims.d[0]; // [S, B]: what the legacy class keeps as mS
        }
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
    std::vector<uint8_t> encoded() const noexcept
    {
        try
        {
            PluginFieldCollection const* fc = mRuntime->getFieldsToSerialize();
            if (fc)
            {
                return encode(mLayout, *fc, mExtras);
            }
        }
        catch (std::exception const& e)
        {
            if (ILogger* l = getLogger())
            {
                l->log(ILogger::Severity::kERROR, e.what());
            }
        }
        catch (...)
        {
        }
        return {};
    }

    V3Ptr mPlugin;
    IPluginV3OneCore* mCore{};
    IPluginV3OneBuild* mBuild{};
    IPluginV3OneRuntime* mRuntime{};
    char const* mVersion;
    std::string mNamespace;
    int32_t mNbInputs;
    Layout mLayout;
    Extras mExtras;
};

Layout layoutOf(char const* pluginName, char const* legacyVersion)
{
    std::string const name = pluginName;
    int const v = std::atoi(legacyVersion);
    if (name == "CustomSkipLayerNormPluginDynamic")
    {
        return v <= 2 ? Layout::kSKIP : Layout::kSKIP_INTERLEAVED;
    }
    if (name == "CustomEmbLayerNormPluginDynamic")
    {
        return v == 1 ? Layout::kEMB_FIXED : Layout::kEMB_VARSEQLEN;
    }
    return v == 1 ? Layout::kQKV : (v == 2 ? Layout::kQKV_VARSEQLEN : Layout::kQKV_INTERLEAVED);
}

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
        return make(name, fc, TensorRTPhase::kBUILD, Extras{});
    }
    IPluginV2* deserializePlugin(AsciiChar const* name, void const* serialData, size_t serialLength) noexcept override
    {
        try
        {
            FieldStore fs;
            Extras ex;
            decode(layoutOf(mName, mVersion), serialData, serialLength, fs, ex);
            PluginFieldCollection const fc = fs.collection();
            return make(name, &fc, TensorRTPhase::kRUNTIME, ex);
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
    IPluginV2* make(AsciiChar const* name, PluginFieldCollection const* fc, TensorRTPhase phase, Extras ex) noexcept
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
            ex.mtron = std::string(mName) == "CustomEmbLayerNormPluginDynamic" && std::atoi(mVersion) == 3;
            return new LegacyAdapter(std::move(p), mVersion, mNamespace, nbIn, layoutOf(mName, mVersion), ex);
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
