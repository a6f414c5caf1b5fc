// CustomEmbLayerNormPluginDynamic, versions 6 (fixed [S,B] inputs, second output = mask index or
// packed mask), 4 (HFace: packed tokens + cu_seqlens) and 5 (MTron: additionally returns the
// pre-LayerNorm embedding sum).
//
// Behaviour follows plugin/embLayerNormPlugin/embLayerNormPlugin.cpp (:42-535, creator :539-690) and
// plugin/embLayerNormPlugin/embLayerNormVarSeqlenPlugin.cpp (:40-712, creators :716-830).
#include "plugin_base.h"

namespace trtamd
{
namespace plugin
{
namespace
{

constexpr char const* kNAME = "CustomEmbLayerNormPluginDynamic";
constexpr char const* kBETA = "bert_embeddings_layernorm_beta";
constexpr char const* kGAMMA = "bert_embeddings_layernorm_gamma";
constexpr char const* kWORD = "bert_embeddings_word_embeddings";
constexpr char const* kTOK = "bert_embeddings_token_type_embeddings";
constexpr char const* kPOS = "bert_embeddings_position_embeddings";

// The five weight tensors every version carries: beta/gamma in binary32, tables in the output type.
struct EmbeddingWeights
{
    HostWeights beta, gamma, word, pos, tok;
    DeviceBuffer betaDev, gammaDev, wordDev, posDev, tokDev;
    int32_t ld{0};
    int32_t wordVocab{0}, posVocab{0}, tokVocab{0};

    void init(DataType type, Weights const& b, Weights const& g, Weights const& w, Weights const& p, Weights const& t)
    {
        ld = static_cast<int32_t>(b.count);
        TRTAMD_VALIDATE(b.count == g.count);
        TRTAMD_VALIDATE(ld > 0);
        TRTAMD_VALIDATE(w.count % ld == 0);
        TRTAMD_VALIDATE(p.count % ld == 0);
        TRTAMD_VALIDATE(t.count % ld == 0);
        wordVocab = static_cast<int32_t>(w.count / ld);
        posVocab = static_cast<int32_t>(p.count / ld);
        tokVocab = static_cast<int32_t>(t.count / ld);
        beta.assign(b, DataType::kFLOAT);
        gamma.assign(g, DataType::kFLOAT);
        word.assign(w, type);
        tok.assign(t, type);
        pos.assign(p, type);
        gammaDev.upload(gamma);
        betaDev.upload(beta);
        wordDev.upload(word);
        posDev.upload(pos);
        tokDev.upload(tok);
    }

    void requireOnDevice() const
    {
        TRTAMD_VALIDATE_MSG(betaDev.get() && gammaDev.get() && wordDev.get() && posDev.get() && tokDev.get(),
            "parameters are not on the device (no GPU was visible when the plugin was created)");
    }

    void serialize(FieldList& f, bool fp16) const
    {
        f.add(kBETA, beta.data(), PluginFieldType::kFLOAT32, static_cast<int32_t>(beta.count()));
        f.add(kGAMMA, gamma.data(), PluginFieldType::kFLOAT32, static_cast<int32_t>(gamma.count()));
        PluginFieldType const ft = fp16 ? PluginFieldType::kFLOAT16 : PluginFieldType::kFLOAT32;
        f.add(kWORD, word.data(), ft, static_cast<int32_t>(word.count()));
        f.add(kTOK, tok.data(), ft, static_cast<int32_t>(tok.count()));
        f.add(kPOS, pos.data(), ft, static_cast<int32_t>(pos.count()));
    }
};

// Reads the five weight fields; returns output_fp16.
bool readEmbeddingFields(PluginFieldCollection const* fc, Weights& beta, Weights& gamma, Weights& word, Weights& pos,
    Weights& tok)
{
    validateRequiredFields({kBETA, kGAMMA, kWORD, kTOK, kPOS}, fc);
    readWeights(fc, kBETA, beta);
    readWeights(fc, kGAMMA, gamma);
    readWeights(fc, kWORD, word);
    readWeights(fc, kTOK, tok);
    readWeights(fc, kPOS, pos);
    bool fp16 = false;
    if (PluginField const* f = findField(fc, "output_fp16"))
    {
        TRTAMD_VALIDATE(f->type == PluginFieldType::kINT32);
        TRTAMD_VALIDATE(f->data != nullptr);
        fp16 = static_cast<int32_t const*>(f->data)[0] != 0;
    }
    return fp16;
}

// ------------------------------------------------------------------------------------------
// version 6
// ------------------------------------------------------------------------------------------
class EmbLayerNormPlugin final : public BertPluginBase
{
public:
    EmbLayerNormPlugin(std::string const& name, DataType type, DataType mhaType, Weights const& beta,
        Weights const& gamma, Weights const& word, Weights const& pos, Weights const& tok, bool useFullMask)
        : BertPluginBase(name, kNAME, "6", 3, 2)
        , mType(type)
        , mMhaType(mhaType)
    {
        mW.init(type, beta, gamma, word, pos, tok);
        mSM = getSmVersion();
        mOutputFp16 = mType == DataType::kHALF ? 1 : 0;
        mUseFullMask = useFullMask ? 1 : 0;
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        auto p = std::make_unique<EmbLayerNormPlugin>(mLayerName, mType, mMhaType, mW.beta.view(), mW.gamma.view(),
            mW.word.view(), mW.pos.view(), mW.tok.view(), mUseFullMask == 1);
        p->mS = mS;
        return p;
    }

    void doOutputTypes(DataType* outputTypes, DataType const*) const override
    {
        TRTAMD_VALIDATE(mType == DataType::kHALF || mType == DataType::kFLOAT);
        outputTypes[0] = mType;
        outputTypes[1] = DataType::kINT32;
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) override
    {
        TRTAMD_VALIDATE(inputs[0].nbDims == 2);
        TRTAMD_VALIDATE(inputs[0].nbDims == inputs[1].nbDims);
        TRTAMD_VALIDATE(inputs[0].nbDims == inputs[2].nbDims);
        outputs[0].nbDims = 5;
        outputs[0].d[0] = inputs[0].d[0];
        outputs[0].d[1] = inputs[0].d[1];
        outputs[0].d[2] = eb.constant(mW.ld);
        outputs[0].d[3] = eb.constant(1);
        outputs[0].d[4] = eb.constant(1);

        outputs[1].nbDims = 2;
        outputs[1].d[0] = inputs[0].d[kBDIM];
        IDimensionExpr const* unfused = eb.constant(kUnfusedMaskSize);
        bool const precisionOk = mMhaType == DataType::kHALF || mMhaType == DataType::kINT8;
        bool const smOk = getMHAMaskPackedSize(mSM, DataType::kHALF, 128) != kUnfusedMaskSize;
        if (mUseFullMask || (smOk && precisionOk))
        {
            // size(S) = 512 for S in {64,96,128}, 6144 for S = 384, otherwise 1: a sum of
            // (S == s) * size(s) terms, plus (sum == 0) * 1
            IDimensionExpr const* S = inputs[0].d[kSDIM];
            struct Case
            {
                int32_t s, size;
            };
            Case const cases[] = {{128, kPackedMaskSize128}, {384, kPackedMaskSize384}, {64, kPackedMaskSize128},
                {96, kPackedMaskSize128}};
            IDimensionExpr const* total = eb.constant(0);
            for (Case const& c : cases)
            {
                IDimensionExpr const* is = eb.operation(DimensionOperation::kEQUAL, *S, *eb.constant(c.s));
                IDimensionExpr const* sel = eb.operation(DimensionOperation::kPROD, *is, *eb.constant(c.size));
                total = eb.operation(DimensionOperation::kSUM, *total, *sel);
            }
            IDimensionExpr const* isZero = eb.operation(DimensionOperation::kEQUAL, *total, *eb.constant(0));
            IDimensionExpr const* sel0 = eb.operation(DimensionOperation::kPROD, *isZero, *unfused);
            outputs[1].d[1] = eb.operation(DimensionOperation::kSUM, *total, *sel0);
        }
        else
        {
            outputs[1].d[1] = unfused;
        }
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        PluginTensorDesc const& desc = inOut[pos].desc;
        if (desc.format != TensorFormat::kLINEAR)
        {
            return false;
        }
        if (pos == 0)
        {
            return desc.type == DataType::kINT32 && desc.dims.nbDims == 2;
        }
        PluginTensorDesc const& prev = inOut[pos - 1].desc;
        if (pos == 1 || pos == 2)
        {
            return desc.type == DataType::kINT32 && desc.dims.nbDims == 2 && desc.dims.d[kBDIM] == prev.dims.d[kBDIM]
                && desc.dims.d[kSDIM] == prev.dims.d[kSDIM];
        }
        if (pos == 3)
        {
            return desc.type == mType && desc.dims.nbDims == 5 && desc.dims.d[kBDIM] == prev.dims.d[kBDIM]
                && desc.dims.d[kSDIM] == prev.dims.d[kSDIM] && desc.dims.d[3] == 1 && desc.dims.d[4] == 1;
        }
        return desc.type == DataType::kINT32;
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const* out) override
    {
        TRTAMD_VALIDATE(in[0].dims.nbDims == 2);
        int64_t const S = in[0].dims.d[kSDIM];
        int64_t const B = in[0].dims.d[kBDIM];
        mS = static_cast<int32_t>(S);
        TRTAMD_VALIDATE(S == in[1].dims.d[kSDIM] && B == in[1].dims.d[kBDIM]);
        TRTAMD_VALIDATE(S == in[2].dims.d[kSDIM] && B == in[2].dims.d[kBDIM]);
        TRTAMD_VALIDATE(out[0].dims.nbDims == 5);
        TRTAMD_VALIDATE(out[0].dims.d[kSDIM] == S && out[0].dims.d[kBDIM] == B);
        TRTAMD_VALIDATE(out[0].dims.d[2] == mW.ld);
        TRTAMD_VALIDATE(out[0].dims.d[3] == 1 && out[0].dims.d[4] == 1);
        if (mUseFullMask)
        {
            TRTAMD_VALIDATE(out[1].dims.nbDims == 2);
            TRTAMD_VALIDATE(out[1].dims.d[0] == B);
            TRTAMD_VALIDATE(out[1].dims.d[1] == -1 || out[1].dims.d[1] == kPackedMaskSize384
                || out[1].dims.d[1] == kPackedMaskSize128);
        }
        else if (S != -1 && B != -1)
        {
            TRTAMD_VALIDATE(out[1].dims.nbDims == 2);
            TRTAMD_VALIDATE(out[1].dims.d[0] == B);
            int32_t const packed = getMHAMaskPackedSize(mSM, mMhaType, static_cast<int32_t>(S));
            TRTAMD_VALIDATE(out[1].dims.d[1] == -1 || out[1].dims.d[1] == packed);
        }
        TRTAMD_VALIDATE(in[0].type == DataType::kINT32 && in[1].type == DataType::kINT32
            && in[2].type == DataType::kINT32);
        TRTAMD_VALIDATE(out[0].type == mType);
        TRTAMD_VALIDATE(out[1].type == DataType::kINT32);
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const*, void const* const* inputs,
        void* const* outputs, void*, hipStream_t stream) override
    {
        int32_t const B = static_cast<int32_t>(inputDesc[0].dims.d[kBDIM]);
        int32_t const S = static_cast<int32_t>(inputDesc[0].dims.d[kSDIM]);
        mW.requireOnDevice();
        auto const* ids = static_cast<int32_t const*>(inputs[0]);
        auto const* segs = static_cast<int32_t const*>(inputs[1]);
        auto const* mask = static_cast<int32_t const*>(inputs[2]);
        int32_t status;
        if (mType == DataType::kFLOAT)
        {
            status = trtamd_emb_layer_norm_fp32(stream, mW.ld, B, S, ids, segs, mW.betaDev.as<float>(),
                mW.gammaDev.as<float>(), mW.wordDev.as<float>(), mW.posDev.as<float>(), mW.tokDev.as<float>(),
                mW.wordVocab, mW.tokVocab, static_cast<float*>(outputs[0]));
        }
        else if (mType == DataType::kHALF)
        {
            status = trtamd_emb_layer_norm_fp16(stream, mW.ld, B, S, ids, segs, mW.betaDev.as<float>(),
                mW.gammaDev.as<float>(), mW.wordDev.as<uint16_t>(), mW.posDev.as<uint16_t>(),
                mW.tokDev.as<uint16_t>(), mW.wordVocab, mW.tokVocab, static_cast<uint16_t*>(outputs[0]));
        }
        else
        {
            logMessage(ILogger::Severity::kERROR,
                "Unsupported type error, expected [kHALF,kFLOAT], but received "
                    + std::to_string(static_cast<int32_t>(mType)));
            return kSTATUS_NOT_SUPPORTED;
        }
        if (status != 0)
        {
            return status;
        }
        // packed mask when the attention plugin downstream runs a fused kernel at this S, else the
        // index of the first masked position per sequence
        if (mUseFullMask || getMHAMaskPackedSize(mSM, mMhaType, S) != kUnfusedMaskSize)
        {
            uint32_t warpsM = 0, warpsN = 0;
            if (S == 64 || S == 96 || S == 128)
            {
                warpsM = 2;
                warpsN = 2;
            }
            else if (S == 384)
            {
                warpsM = 1;
                warpsN = 8;
            }
            return trtamd_convert_mask(static_cast<uint32_t>(S), static_cast<uint32_t>(B), warpsM, warpsN, 1, mask,
                static_cast<uint32_t*>(outputs[1]), stream);
        }
        return trtamd_compute_mask_idx(stream, S, B, mask, static_cast<int32_t*>(outputs[1]));
    }

    void doSerialize(FieldList& f) override
    {
        f.add("output_fp16", &mOutputFp16, PluginFieldType::kINT32, 1);
        f.add("full_mask", &mUseFullMask, PluginFieldType::kINT32, 1);
        f.add("mha_type_id", &mMhaType, PluginFieldType::kINT32, 1);
        mW.serialize(f, mOutputFp16 != 0);
    }

private:
    EmbeddingWeights mW;
    DataType mType;
    DataType mMhaType;
    int32_t mSM{0};
    int32_t mS{0};
    int32_t mOutputFp16{0};
    int32_t mUseFullMask{0};
};

class EmbLayerNormCreator final : public BertCreatorBase
{
public:
    EmbLayerNormCreator()
        : BertCreatorBase(kNAME, "6",
            {PluginField(kBETA), PluginField(kGAMMA), PluginField(kWORD), PluginField(kTOK), PluginField(kPOS),
                PluginField("output_fp16"), PluginField("full_mask"), PluginField("mha_type_id")})
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc, TensorRTPhase) override
    {
        Weights beta{}, gamma{}, word{}, pos{}, tok{};
        bool const fp16 = readEmbeddingFields(fc, beta, gamma, word, pos, tok);
        bool fullMask = false;
        if (PluginField const* f = findField(fc, "full_mask"))
        {
            TRTAMD_VALIDATE(f->type == PluginFieldType::kINT32);
            TRTAMD_VALIDATE(f->data != nullptr);
            fullMask = static_cast<int32_t const*>(f->data)[0] != 0;
        }
        int32_t mhaTypeId = 0;
        if (readScalar(fc, "mha_type_id", mhaTypeId))
        {
            TRTAMD_VALIDATE(mhaTypeId >= 0 && mhaTypeId <= 3);
        }
        return std::make_unique<EmbLayerNormPlugin>(name, fp16 ? DataType::kHALF : DataType::kFLOAT,
            static_cast<DataType>(mhaTypeId), beta, gamma, word, pos, tok, fullMask);
    }
};

// ------------------------------------------------------------------------------------------
// versions 4 (HFace) and 5 (MTron)
// ------------------------------------------------------------------------------------------
class EmbLayerNormVarSeqlenPlugin final : public BertPluginBase
{
public:
    EmbLayerNormVarSeqlenPlugin(std::string const& name, bool mtron, DataType type, Weights const& beta,
        Weights const& gamma, Weights const& word, Weights const& pos, Weights const& tok)
        : BertPluginBase(name, kNAME, mtron ? "5" : "4", 4, 2)
        , mMtron(mtron)
        , mType(type)
        , mMaskType(mtron ? type : DataType::kINT32)
    {
        mW.init(type, beta, gamma, word, pos, tok);
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        return std::make_unique<EmbLayerNormVarSeqlenPlugin>(mLayerName, mMtron, mType, mW.beta.view(),
            mW.gamma.view(), mW.word.view(), mW.pos.view(), mW.tok.view());
    }

    void doOutputTypes(DataType* outputTypes, DataType const*) const override
    {
        TRTAMD_VALIDATE(mType == DataType::kHALF || mType == DataType::kFLOAT);
        outputTypes[0] = mType;
        outputTypes[1] = mMaskType;
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) override
    {
        TRTAMD_VALIDATE(inputs[0].nbDims == 1); // sum of all sequence lengths
        TRTAMD_VALIDATE(inputs[0].nbDims == inputs[1].nbDims);
        TRTAMD_VALIDATE(inputs[2].nbDims == 1); // B + 1
        outputs[0].nbDims = 4;
        outputs[0].d[0] = inputs[0].d[0];
        outputs[0].d[1] = eb.constant(mW.ld);
        outputs[0].d[2] = eb.constant(1);
        outputs[0].d[3] = eb.constant(1);
        if (mMtron)
        {
            outputs[1] = outputs[0]; // the residual stream: the embedding sum before LayerNorm
        }
        else
        {
            outputs[1].nbDims = 0; // an empty tensor kept for backward compatibility
        }
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        PluginTensorDesc const& desc = inOut[pos].desc;
        if (desc.format != TensorFormat::kLINEAR)
        {
            return false;
        }
        if (pos == 0 || pos == 2) // input_ids and cu_seqlens
        {
            return desc.type == DataType::kINT32 && desc.dims.nbDims == 1;
        }
        PluginTensorDesc const& prev = inOut[pos - 1].desc;
        if (pos == 1) // segment ids: same extent as input_ids
        {
            return desc.type == DataType::kINT32 && desc.dims.nbDims == 1 && desc.dims.d[0] == prev.dims.d[0];
        }
        if (pos == 3) // dummy tensor whose extent is the maximum sequence length
        {
            return desc.dims.nbDims == 1;
        }
        if (pos == mNbInputs)
        {
            return desc.type == mType && desc.dims.nbDims == 4 && desc.dims.d[0] == inOut[0].desc.dims.d[0]
                && desc.dims.d[2] == 1 && desc.dims.d[3] == 1;
        }
        return desc.type == mMaskType;
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const* out) override
    {
        TRTAMD_VALIDATE(in[0].dims.nbDims == 1);
        TRTAMD_VALIDATE(in[1].dims.nbDims == 1);
        TRTAMD_VALIDATE(in[1].dims.d[0] == in[0].dims.d[0]);
        TRTAMD_VALIDATE(in[2].dims.nbDims == 1);
        TRTAMD_VALIDATE(out[0].dims.nbDims == 4);
        TRTAMD_VALIDATE(out[0].dims.d[0] == in[0].dims.d[0]);
        TRTAMD_VALIDATE(out[0].dims.d[2] == 1 && out[0].dims.d[3] == 1);
        TRTAMD_VALIDATE(in[0].type == DataType::kINT32 && in[1].type == DataType::kINT32
            && in[2].type == DataType::kINT32);
        TRTAMD_VALIDATE(out[0].dims.d[1] == mW.ld);
        TRTAMD_VALIDATE(out[0].type == mType);
        if (mMtron)
        {
            TRTAMD_VALIDATE(out[1].dims.nbDims == 4);
            TRTAMD_VALIDATE(out[1].dims.d[0] == in[0].dims.d[0]);
            TRTAMD_VALIDATE(out[1].dims.d[1] == mW.ld);
            TRTAMD_VALIDATE(out[1].dims.d[2] == 1 && out[1].dims.d[3] == 1);
        }
        else
        {
            TRTAMD_VALIDATE(out[1].dims.nbDims == 0);
        }
        TRTAMD_VALIDATE(out[1].type == mMaskType);
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const*, void const* const* inputs,
        void* const* outputs, void*, hipStream_t stream) override
    {
        int32_t const B = static_cast<int32_t>(inputDesc[2].dims.d[0]) - 1;
        // the maximum sequence length is the extent of the dummy input
        int32_t const maxSeqlen = static_cast<int32_t>(inputDesc[3].dims.d[0]);
        // The reference launches one of four grids (128, 192, 256, 384 positions per sequence) and
        // never looks at positions beyond 384; here longer sequences are simply covered.
        int32_t S = maxSeqlen <= 128 ? 128 : maxSeqlen <= 192 ? 192 : maxSeqlen <= 256 ? 256 : 384;
        if (maxSeqlen > S)
        {
            S = maxSeqlen;
        }
        mW.requireOnDevice();
        auto const* ids = static_cast<int32_t const*>(inputs[0]);
        auto const* segs = static_cast<int32_t const*>(inputs[1]);
        auto const* cu = static_cast<int32_t const*>(inputs[2]);
        if (mType == DataType::kFLOAT)
        {
            auto* out = static_cast<float*>(outputs[0]);
            return mMtron
                ? trtamd_emb_layer_norm_mtron_fp32(stream, mW.ld, B, S, ids, segs, cu, mW.betaDev.as<float>(),
                    mW.gammaDev.as<float>(), mW.wordDev.as<float>(), mW.posDev.as<float>(), mW.tokDev.as<float>(),
                    mW.wordVocab, mW.tokVocab, out, static_cast<float*>(outputs[1]))
                : trtamd_emb_layer_norm_hface_fp32(stream, mW.ld, B, S, ids, segs, cu, mW.betaDev.as<float>(),
                    mW.gammaDev.as<float>(), mW.wordDev.as<float>(), mW.posDev.as<float>(), mW.tokDev.as<float>(),
                    mW.wordVocab, mW.tokVocab, out);
        }
        if (mType == DataType::kHALF)
        {
            auto* out = static_cast<uint16_t*>(outputs[0]);
            return mMtron
                ? trtamd_emb_layer_norm_mtron_fp16(stream, mW.ld, B, S, ids, segs, cu, mW.betaDev.as<float>(),
                    mW.gammaDev.as<float>(), mW.wordDev.as<uint16_t>(), mW.posDev.as<uint16_t>(),
                    mW.tokDev.as<uint16_t>(), mW.wordVocab, mW.tokVocab, out, static_cast<uint16_t*>(outputs[1]))
                : trtamd_emb_layer_norm_hface_fp16(stream, mW.ld, B, S, ids, segs, cu, mW.betaDev.as<float>(),
                    mW.gammaDev.as<float>(), mW.wordDev.as<uint16_t>(), mW.posDev.as<uint16_t>(),
                    mW.tokDev.as<uint16_t>(), mW.wordVocab, mW.tokVocab, out);
        }
        logMessage(ILogger::Severity::kERROR,
            "Unsupported type error, expected [kHALF,kFLOAT], but received "
                + std::to_string(static_cast<int32_t>(mType)));
        return kSTATUS_NOT_SUPPORTED;
    }

    void doSerialize(FieldList& f) override
    {
        mOutputFp16 = mType == DataType::kHALF ? 1 : 0;
        f.add("output_fp16", &mOutputFp16, PluginFieldType::kINT32, 1);
        mW.serialize(f, mOutputFp16 != 0);
    }

private:
    bool const mMtron;
    DataType mType;
    DataType mMaskType;
    int32_t mOutputFp16{0};
    EmbeddingWeights mW;
};

class EmbLayerNormVarSeqlenCreator : public BertCreatorBase
{
public:
    explicit EmbLayerNormVarSeqlenCreator(bool mtron)
        : BertCreatorBase(kNAME, mtron ? "5" : "4",
            {PluginField("output_fp16", nullptr, PluginFieldType::kINT32, 1),
                PluginField(kBETA, nullptr, PluginFieldType::kFLOAT32, 0),
                PluginField(kGAMMA, nullptr, PluginFieldType::kFLOAT32, 0),
                PluginField(kWORD, nullptr, PluginFieldType::kUNKNOWN, 0),
                PluginField(kTOK, nullptr, PluginFieldType::kUNKNOWN, 0),
                PluginField(kPOS, nullptr, PluginFieldType::kUNKNOWN, 0)})
        , mMtron(mtron)
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc, TensorRTPhase) override
    {
        Weights beta{}, gamma{}, word{}, pos{}, tok{};
        bool const fp16 = readEmbeddingFields(fc, beta, gamma, word, pos, tok);
        return std::make_unique<EmbLayerNormVarSeqlenPlugin>(name, mMtron, fp16 ? DataType::kHALF : DataType::kFLOAT,
            beta, gamma, word, pos, tok);
    }

private:
    bool const mMtron;
};

struct EmbLayerNormHFaceCreator : EmbLayerNormVarSeqlenCreator
{
    EmbLayerNormHFaceCreator()
        : EmbLayerNormVarSeqlenCreator(false)
    {
    }
};
struct EmbLayerNormMTronCreator : EmbLayerNormVarSeqlenCreator
{
    EmbLayerNormMTronCreator()
        : EmbLayerNormVarSeqlenCreator(true)
    {
    }
};

REGISTER_TENSORRT_PLUGIN(EmbLayerNormCreator);
REGISTER_TENSORRT_PLUGIN(EmbLayerNormHFaceCreator);
REGISTER_TENSORRT_PLUGIN(EmbLayerNormMTronCreator);

} // namespace
} // namespace plugin
} // namespace trtamd
