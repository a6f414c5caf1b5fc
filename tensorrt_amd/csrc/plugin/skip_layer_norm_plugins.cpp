// CustomSkipLayerNormPluginDynamic, versions 5, 6 (linear layouts, FP32/FP16/INT8) and
// 7, 8 (INT8, 32-interleaved; 8 also emits the quantised pre-LayerNorm sum).
//
// Behaviour follows plugin/skipLayerNormPlugin/skipLayerNormPlugin.cpp (SkipLayerNormPluginV3 :44-437,
// SkipLayerNormVarSeqlenPluginV3 :554-938, creators :441-551, :942-1045) and
// plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedPlugin.cpp (:41-488, creators :492-600).
#include "plugin_base.h"

#include <algorithm>

namespace trtamd
{
namespace plugin
{
namespace
{

constexpr char const* kNAME = "CustomSkipLayerNormPluginDynamic";

// ------------------------------------------------------------------------------------------
// versions 5 and 6
// ------------------------------------------------------------------------------------------
class SkipLayerNormPlugin final : public BertPluginBase
{
public:
    // fixedShape = version 5: [S,B,E,1,1] inputs, `ld` attribute; version 6: any equal shapes,
    // ld = number of beta elements.
    SkipLayerNormPlugin(std::string const& name, bool fixedShape, DataType type, int32_t ld, Weights const& beta,
        Weights const& gamma, Weights const& bias)
        : BertPluginBase(name, kNAME, fixedShape ? "5" : "6", 2, 1)
        , mFixedShape(fixedShape)
        , mType(type)
        , mLd(ld)
    {
        TRTAMD_VALIDATE(mType == DataType::kFLOAT || mType == DataType::kHALF || mType == DataType::kINT8);
        if (!mFixedShape)
        {
            TRTAMD_VALIDATE(mLd > 0);
            TRTAMD_VALIDATE(beta.count == gamma.count);
        }
        // parameters are binary16 when the tensors are INT8
        mCfgType = mType == DataType::kINT8 ? DataType::kHALF : mType;
        mBeta.assign(beta, mCfgType);
        mGamma.assign(gamma, mCfgType);
        mHasBias = bias.values != nullptr;
        if (mHasBias)
        {
            mBias.assign(bias, mCfgType);
        }
        mBetaDev.upload(mBeta);
        mGammaDev.upload(mGamma);
        if (mHasBias)
        {
            mBiasDev.upload(mBias);
        }
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        Weights const none{DataType::kFLOAT, nullptr, 0};
        return std::make_unique<SkipLayerNormPlugin>(
            mLayerName, mFixedShape, mType, mLd, mBeta.view(), mGamma.view(), mHasBias ? mBias.view() : none);
    }

    void doOutputTypes(DataType* outputTypes, DataType const* inputTypes) const override
    {
        outputTypes[0] = inputTypes[0];
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder&) override
    {
        TRTAMD_VALIDATE(inputs[0].nbDims == inputs[1].nbDims);
        outputs[0] = inputs[0];
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        PluginTensorDesc const& in = inOut[pos].desc;
        if (!mFixedShape && in.type != mType)
        {
            return false;
        }
        if (pos == 0)
        {
            if (mType == DataType::kINT8)
            {
                // the trailing dimensions are 1, so any CHWx vectorisation is byte-linear
                TensorFormat const fmt = mLd < 32 ? TensorFormat::kCHW4 : TensorFormat::kCHW32;
                return in.type == mType && in.format == fmt;
            }
            return in.type == mType && in.format == TensorFormat::kLINEAR;
        }
        PluginTensorDesc const& prev = inOut[pos - 1].desc;
        return in.type == prev.type && in.format == prev.format;
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const*) override
    {
        if (mType == DataType::kFLOAT || mType == DataType::kHALF)
        {
            TRTAMD_VALIDATE(mType == in[0].type);
            TRTAMD_VALIDATE(mType == in[1].type);
        }
        else
        {
            TRTAMD_VALIDATE(mType == in[0].type || DataType::kFLOAT == in[0].type);
            TRTAMD_VALIDATE(mType == in[1].type || DataType::kFLOAT == in[1].type);
        }
        Dims const& d0 = in[0].dims;
        Dims const& d1 = in[1].dims;
        TRTAMD_VALIDATE(d0.nbDims == d1.nbDims);
        TRTAMD_VALIDATE(std::equal(d0.d, d0.d + d0.nbDims, d1.d));
        if (mFixedShape)
        {
            TRTAMD_VALIDATE(d0.nbDims == 5);
            mLd = static_cast<int32_t>(d0.d[kHDIM]);
            TRTAMD_VALIDATE(mLd != 0);
            TRTAMD_VALIDATE(d0.d[3] == 1);
            TRTAMD_VALIDATE(d0.d[4] == 1);
        }
        mCfgType = in[0].type == DataType::kINT8 ? DataType::kHALF : in[0].type;
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void*, hipStream_t stream) override
    {
        int64_t const n = volume(inputDesc[0].dims);
        if (!mFixedShape)
        {
            TRTAMD_VALIDATE_MSG(n % mLd == 0, "inconsistent dimensions");
        }
        requireParameters();
        DataType const iType = inputDesc[0].type;
        void const* bias = mHasBias ? mBiasDev.get() : nullptr;
        if (iType == DataType::kFLOAT)
        {
            return trtamd_skip_layer_norm_fp32(stream, mLd, n, static_cast<float const*>(inputs[0]),
                static_cast<float const*>(inputs[1]), mBetaDev.as<float>(), mGammaDev.as<float>(),
                static_cast<float*>(outputs[0]), static_cast<float const*>(bias));
        }
        if (iType == DataType::kHALF)
        {
            return trtamd_skip_layer_norm_fp16(stream, mLd, n, static_cast<uint16_t const*>(inputs[0]),
                static_cast<uint16_t const*>(inputs[1]), mBetaDev.as<uint16_t>(), mGammaDev.as<uint16_t>(),
                static_cast<uint16_t*>(outputs[0]), static_cast<uint16_t const*>(bias));
        }
        if (iType == DataType::kINT8)
        {
            TRTAMD_VALIDATE(outputDesc[0].scale != 0.0F);
            return trtamd_skip_layer_norm_dqq(stream, mLd, n, static_cast<int8_t const*>(inputs[0]),
                static_cast<int8_t const*>(inputs[1]), mBetaDev.as<uint16_t>(), mGammaDev.as<uint16_t>(),
                static_cast<int8_t*>(outputs[0]), static_cast<uint16_t const*>(bias), inputDesc[0].scale,
                inputDesc[1].scale, 1.F / outputDesc[0].scale);
        }
        throw PluginError("Unsupported type error, expected [kINT8,kHALF,kFLOAT], but received "
            + std::to_string(static_cast<int32_t>(iType)));
    }

    void doSerialize(FieldList& f) override
    {
        f.add("type_id", &mType, PluginFieldType::kINT32, 1);
        f.add("ld", &mLd, PluginFieldType::kINT32, 1);
        PluginFieldType const ft = mCfgType == DataType::kHALF ? PluginFieldType::kFLOAT16 : PluginFieldType::kFLOAT32;
        TRTAMD_VALIDATE(mBeta.type() == mCfgType && mGamma.type() == mCfgType);
        f.add("beta", mBeta.data(), ft, static_cast<int32_t>(mBeta.count()));
        f.add("gamma", mGamma.data(), ft, static_cast<int32_t>(mGamma.count()));
        if (mHasBias)
        {
            f.add("bias", mBias.data(), ft, static_cast<int32_t>(mBias.count()));
        }
    }

private:
    void requireParameters() const
    {
        TRTAMD_VALIDATE_MSG(mBetaDev.get() && mGammaDev.get() && (!mHasBias || mBiasDev.get()),
            "parameters are not on the device (no GPU was visible when the plugin was created)");
        TRTAMD_VALIDATE_MSG(mBeta.count() >= mLd && mGamma.count() >= mLd && (!mHasBias || mBias.count() >= mLd),
            "beta/gamma/bias hold fewer than ld elements");
    }

    bool const mFixedShape;
    DataType mType;
    DataType mCfgType;
    int32_t mLd;
    bool mHasBias{false};
    HostWeights mBeta, mGamma, mBias;
    DeviceBuffer mBetaDev, mGammaDev, mBiasDev;
};

class SkipLayerNormCreator : public BertCreatorBase
{
public:
    explicit SkipLayerNormCreator(bool fixedShape)
        : BertCreatorBase(kNAME, fixedShape ? "5" : "6",
            fixedShape ? std::vector<PluginField>{PluginField("type_id"), PluginField("ld"), PluginField("beta"),
                PluginField("gamma"), PluginField("bias")}
                       : std::vector<PluginField>{PluginField("type_id"), PluginField("beta"), PluginField("gamma"),
                           PluginField("bias")})
        , mFixedShape(fixedShape)
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc, TensorRTPhase) override
    {
        if (mFixedShape)
        {
            validateRequiredFields({"type_id", "beta", "ld", "gamma"}, fc);
        }
        else
        {
            validateRequiredFields({"type_id", "beta", "gamma"}, fc);
        }
        int32_t typeId = -1;
        int32_t ld = 0;
        Weights beta{DataType::kFLOAT, nullptr, 0};
        Weights gamma{DataType::kFLOAT, nullptr, 0};
        Weights bias{DataType::kFLOAT, nullptr, 0};
        readScalar(fc, "type_id", typeId);
        readScalar(fc, "ld", ld);
        readWeights(fc, "beta", beta);
        readWeights(fc, "gamma", gamma);
        readWeights(fc, "bias", bias);
        TRTAMD_VALIDATE_MSG(typeId >= 0 && typeId <= 3, "SkipLayerNorm: Invalid type ID: " + std::to_string(typeId));
        TRTAMD_VALIDATE_MSG(beta.values != nullptr, "SkipLayerNorm: invalid beta");
        TRTAMD_VALIDATE_MSG(beta.count > 0, "SkipLayerNorm: invalid beta");
        TRTAMD_VALIDATE_MSG(gamma.values != nullptr, "SkipLayerNorm: invalid gamma");
        TRTAMD_VALIDATE_MSG(gamma.count > 0, "SkipLayerNorm: invalid gamma");
        if (bias.values != nullptr)
        {
            TRTAMD_VALIDATE_MSG(bias.count > 0, "SkipLayerNorm: invalid bias");
        }
        if (!mFixedShape)
        {
            ld = static_cast<int32_t>(beta.count);
        }
        return std::make_unique<SkipLayerNormPlugin>(name, mFixedShape, static_cast<DataType>(typeId), ld, beta, gamma,
            bias);
    }

private:
    bool const mFixedShape;
};

// ------------------------------------------------------------------------------------------
// versions 7 (HFace) and 8 (MTron): INT8, [1,E,T,1] in TensorFormat::kCHW32
// ------------------------------------------------------------------------------------------
class SkipLayerNormInterleavedPlugin final : public BertPluginBase
{
public:
    // onDevice: put gamma and beta on the device now.  Runtime-phase objects (and their clones) do, so that neither
    // onShapeChange nor enqueue ever allocates or copies for them; build-phase objects, which may never run, wait
    // for their first shape change as the reference does.
    SkipLayerNormInterleavedPlugin(std::string const& name, bool mtron, Weights const& beta, Weights const& gamma,
        bool onDevice)
        : BertPluginBase(name, kNAME, mtron ? "8" : "7", 2, mtron ? 2 : 1)
        , mMtron(mtron)
        , mLd(static_cast<int32_t>(beta.count))
    {
        TRTAMD_VALIDATE(mLd > 0);
        TRTAMD_VALIDATE(beta.count == gamma.count);
        mBeta.assign(beta, DataType::kHALF);
        mGamma.assign(gamma, DataType::kHALF);
        if (onDevice)
        {
            uploadParams();
        }
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        return std::make_unique<SkipLayerNormInterleavedPlugin>(mLayerName, mMtron, mBeta.view(), mGamma.view(),
            mParamsOnDevice);
    }

    void doOutputTypes(DataType* outputTypes, DataType const* inputTypes) const override
    {
        for (int32_t i = 0; i < mNbOutputs; ++i)
        {
            outputTypes[i] = inputTypes[0];
        }
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder&) override
    {
        TRTAMD_VALIDATE(inputs[0].nbDims == inputs[1].nbDims);
        for (int32_t i = 0; i < mNbOutputs; ++i)
        {
            outputs[i] = inputs[0];
        }
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        PluginTensorDesc const& desc = inOut[pos].desc;
        return desc.type == DataType::kINT8 && desc.format == TensorFormat::kCHW32;
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const*) override
    {
        TRTAMD_VALIDATE(DataType::kINT8 == in[0].type);
        TRTAMD_VALIDATE(DataType::kINT8 == in[1].type);
        Dims const& d0 = in[0].dims;
        Dims const& d1 = in[1].dims;
        TRTAMD_VALIDATE(d0.nbDims == d1.nbDims);
        TRTAMD_VALIDATE(std::equal(d0.d, d0.d + d0.nbDims, d1.d));
        // a build-phase object's parameters go to the device on its first shape change, as in the reference
        uploadParams();
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void*, hipStream_t stream) override
    {
        PluginTensorDesc const& iDesc = inputDesc[0];
        PluginTensorDesc const& sDesc = inputDesc[1];
        PluginTensorDesc const& oDesc = outputDesc[0];
        checkDescs(iDesc, sDesc, oDesc);
        if (mMtron)
        {
            TRTAMD_VALIDATE(std::equal(iDesc.dims.d, iDesc.dims.d + iDesc.dims.nbDims, outputDesc[1].dims.d));
        }
        TRTAMD_VALIDATE_MSG(mBetaDev.get() && mGammaDev.get(), "parameters are not on the device (onShapeChange first)");
        int32_t const ld = static_cast<int32_t>(iDesc.dims.d[1]);
        int32_t const total = static_cast<int32_t>(iDesc.dims.d[2]);
        TRTAMD_VALIDATE_MSG(ld == mLd, "hidden size differs from the number of beta elements");
        float const dqIn = iDesc.scale;
        float const dqSkip = sDesc.scale;
        float const qScale = 1.F / oDesc.scale;
        auto const* input = static_cast<int8_t const*>(inputs[0]);
        auto const* skip = static_cast<int8_t const*>(inputs[1]);
        auto* output = static_cast<int8_t*>(outputs[0]);
        auto const* beta = mBetaDev.as<uint16_t>();
        auto const* gamma = mGammaDev.as<uint16_t>();
        // the reference switches kernels (and with them epsilon and the preln clip) at 4096 tokens
        bool const small = total < 4096;
        if (!mMtron)
        {
            return small
                ? trtamd_skipln_interleaved_small_hface(stream, ld, total, input, skip, beta, gamma, output, dqIn,
                    dqSkip, qScale)
                : trtamd_skipln_interleaved_large_hface(stream, ld, total, input, skip, beta, gamma, output, dqIn,
                    dqSkip, qScale);
        }
        auto* preln = static_cast<int8_t*>(outputs[1]);
        float const qSkipScale = 1.F / outputDesc[1].scale;
        return small ? trtamd_skipln_interleaved_small_mtron(stream, ld, total, input, skip, beta, gamma, output, preln,
                   dqIn, dqSkip, qScale, qSkipScale)
                     : trtamd_skipln_interleaved_large_mtron(stream, ld, total, input, skip, beta, gamma, output, preln,
                         dqIn, dqSkip, qScale, qSkipScale);
    }

    void doSerialize(FieldList& f) override
    {
        f.add("beta", mBeta.data(), PluginFieldType::kFLOAT16, static_cast<int32_t>(mBeta.count()));
        f.add("gamma", mGamma.data(), PluginFieldType::kFLOAT16, static_cast<int32_t>(mGamma.count()));
    }

private:
    void uploadParams()
    {
        if (!mParamsOnDevice)
        {
            mGammaDev.upload(mGamma);
            mBetaDev.upload(mBeta);
            mParamsOnDevice = true;
        }
    }

    static void checkDescs(PluginTensorDesc const& iDesc, PluginTensorDesc const& sDesc, PluginTensorDesc const& oDesc)
    {
        TRTAMD_VALIDATE(iDesc.dims.nbDims == 4);
        TRTAMD_VALIDATE(iDesc.dims.nbDims == sDesc.dims.nbDims);
        TRTAMD_VALIDATE(std::equal(iDesc.dims.d, iDesc.dims.d + iDesc.dims.nbDims, sDesc.dims.d));
        TRTAMD_VALIDATE(std::equal(iDesc.dims.d, iDesc.dims.d + iDesc.dims.nbDims, oDesc.dims.d));
        TRTAMD_VALIDATE(iDesc.dims.d[0] == 1);
        TRTAMD_VALIDATE(iDesc.dims.d[3] == 1);
        TRTAMD_VALIDATE(iDesc.format == TensorFormat::kCHW32);
        TRTAMD_VALIDATE(iDesc.type == DataType::kINT8);
        TRTAMD_VALIDATE(iDesc.format == sDesc.format);
        TRTAMD_VALIDATE(iDesc.format == oDesc.format);
        TRTAMD_VALIDATE(iDesc.type == sDesc.type);
        TRTAMD_VALIDATE(iDesc.type == oDesc.type);
    }

    bool const mMtron;
    int32_t const mLd;
    bool mParamsOnDevice{false};
    HostWeights mBeta, mGamma;
    DeviceBuffer mBetaDev, mGammaDev;
};

class SkipLayerNormInterleavedCreator : public BertCreatorBase
{
public:
    explicit SkipLayerNormInterleavedCreator(bool mtron)
        : BertCreatorBase(kNAME, mtron ? "8" : "7", {PluginField("beta"), PluginField("gamma")})
        , mMtron(mtron)
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc,
        TensorRTPhase phase) override
    {
        validateRequiredFields({"beta", "gamma"}, fc);
        Weights beta{DataType::kFLOAT, nullptr, 0};
        Weights gamma{DataType::kFLOAT, nullptr, 0};
        readWeights(fc, "beta", beta);
        readWeights(fc, "gamma", gamma);
        TRTAMD_VALIDATE_MSG(beta.values != nullptr, "SkipLayerNorm: invalid beta");
        TRTAMD_VALIDATE_MSG(beta.count > 0, "SkipLayerNorm: invalid beta");
        TRTAMD_VALIDATE_MSG(gamma.values != nullptr, "SkipLayerNorm: invalid gamma");
        TRTAMD_VALIDATE_MSG(gamma.count > 0, "SkipLayerNorm: invalid gamma");
        return std::make_unique<SkipLayerNormInterleavedPlugin>(name, mMtron, beta, gamma,
            phase == TensorRTPhase::kRUNTIME);
    }

private:
    bool const mMtron;
};

struct SkipLayerNormV5Creator : SkipLayerNormCreator
{
    SkipLayerNormV5Creator()
        : SkipLayerNormCreator(true)
    {
    }
};
struct SkipLayerNormV6Creator : SkipLayerNormCreator
{
    SkipLayerNormV6Creator()
        : SkipLayerNormCreator(false)
    {
    }
};
struct SkipLayerNormV7Creator : SkipLayerNormInterleavedCreator
{
    SkipLayerNormV7Creator()
        : SkipLayerNormInterleavedCreator(false)
    {
    }
};
struct SkipLayerNormV8Creator : SkipLayerNormInterleavedCreator
{
    SkipLayerNormV8Creator()
        : SkipLayerNormInterleavedCreator(true)
    {
    }
};

REGISTER_TENSORRT_PLUGIN(SkipLayerNormV5Creator);
REGISTER_TENSORRT_PLUGIN(SkipLayerNormV6Creator);
REGISTER_TENSORRT_PLUGIN(SkipLayerNormV7Creator);
REGISTER_TENSORRT_PLUGIN(SkipLayerNormV8Creator);

} // namespace
} // namespace plugin
} // namespace trtamd
