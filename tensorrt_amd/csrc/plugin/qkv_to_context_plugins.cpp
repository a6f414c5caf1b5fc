// CustomQKVToContextPluginDynamic, versions 4 (fixed [S,B,3E,1,1] layout, optional mask),
// 5 (adds packed variable-length input with cu_seqlens) and 6 (INT8, 32-interleaved, cu_seqlens).
//
// Behaviour follows plugin/bertQKVToContextPlugin/qkvToContextPlugin.cpp (QKVToContextPluginDynamic
// :56-579, creator :581-746; QKVToContextVarSeqlenPlugin :762-1353, creator :1355-1500),
// plugin/bertQKVToContextPlugin/qkvToContextInt8InterleavedPlugin.cpp (:49-319, creator :323-470)
// and the runner bookkeeping of plugin/bertQKVToContextPlugin/mhaRunner.{h,cu}.
// The reference picks between precompiled fused kernels and a cuBLAS path; here the same decision
// picks between trtamd_fused_mha_run and trtamd_unfused_mha.
#include "plugin_base.h"

#include <cmath>

namespace trtamd
{
namespace plugin
{
namespace
{

constexpr char const* kNAME = "CustomQKVToContextPluginDynamic";
constexpr int32_t kIIDX = 0; // packed QKV
constexpr int32_t kMIDX = 1; // mask
// CUBLAS_GEMM_DEFAULT_TENSOR_OP, the value the reference's runner holds before it has tuned; here "route by shape"
constexpr int32_t kDefaultGemmAlgo = TRTAMD_UNFUSED_ROUTE_BY_SHAPE;

uint32_t floatBits(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}

uint32_t half2Bits(float f)
{
    uint32_t const h = floatToHalfBits(f);
    return h | (h << 16);
}

// Geometry of MHARunner::setup (plugin/bertQKVToContextPlugin/mhaRunner.h:62-83) plus which
// runner it belongs to; (de)serialised in the reference's byte layout
// (mhaRunner.cu:456-474 for the fused runners, :489-507 for the unfused one).
// The unfused runner's first algorithm slot holds the route that trtamd_unfused_mha_tune found fastest for the configured
// shape (the reference keeps the cuBLAS algorithms of its two batched products there, found the same way at set-up:
// mhaRunner.cu:346-444, 476-487); the second slot has nothing to hold and stays at the default.
struct RunnerState
{
    bool unfused{false};
    bool setUp{false};
    int32_t S{0}, B{0}, headSize{0};
    int32_t algo1{kDefaultGemmAlgo}, algo2{kDefaultGemmAlgo};
    int32_t tunedS{0}, tunedB{0}; // the shape algo1 was timed for (0: never)

    // UnfusedMHARunner::setup's "if (!mIsBestAlgoFound)" step: once per configured shape, at build time, on the
    // device of the calling thread; without a device (or when the timing fails) the route stays with the shape
    void tune(DataType type, int32_t numHeads)
    {
        if (!unfused || !setUp || (tunedS == S && tunedB == B) || type == DataType::kINT8 || !deviceAvailable())
        {
            return;
        }
        int32_t route = kDefaultGemmAlgo;
        if (trtamd_unfused_mha_tune(static_cast<int32_t>(type), S, B, numHeads, headSize, &route, nullptr)
            == TRTAMD_STATUS_SUCCESS)
        {
            algo1 = route;
        }
        else
        {
            logMessage(ILogger::Severity::kWARNING,
                std::string("the unfused attention routes could not be timed: ") + trtamd_last_error());
            algo1 = kDefaultGemmAlgo;
        }
        tunedS = S;
        tunedB = B;
    }
    // what enqueue passes on: a route this library knows, or "by shape" for anything else a stream may hold (the
    // reference writes cuBLAS algorithm numbers there)
    int32_t route() const
    {
        bool const oneLaunch = algo1 == TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH && headSize <= 128;
        return oneLaunch || algo1 == TRTAMD_UNFUSED_ROUTE_THREE_LAUNCHES ? algo1 : TRTAMD_UNFUSED_ROUTE_BY_SHAPE;
    }

    void setup(int32_t s, int32_t b, int32_t d)
    {
        TRTAMD_VALIDATE(s);
        TRTAMD_VALIDATE(b);
        S = s;
        B = b;
        headSize = d;
        setUp = true;
    }
    size_t serializedSize() const
    {
        return (unfused ? 5 : 3) * sizeof(int32_t);
    }
    void serialize(std::vector<uint8_t>& buf) const
    {
        std::vector<int32_t> v;
        if (unfused)
        {
            v = {algo1, algo2, S, B, headSize};
        }
        else
        {
            v = {S, B, headSize};
        }
        buf.resize(v.size() * sizeof(int32_t));
        std::memcpy(buf.data(), v.data(), buf.size());
    }
    // `bytes` = length of the serialised field; a negative value means "not known" (clones, whose buffer was
    // written by serialize() a line earlier)
    void deserialize(void const* data, int64_t bytes = -1)
    {
        TRTAMD_VALIDATE_MSG(bytes < 0 || static_cast<size_t>(bytes) >= serializedSize(),
            "runnerStateBuffer is shorter than the runner state it must hold");
        auto const* v = static_cast<int32_t const*>(data);
        if (unfused)
        {
            algo1 = v[0];
            algo2 = v[1];
            v += 2;
        }
        setup(v[0], v[1], v[2]);
    }
    // UnfusedMHARunner::getWorkspaceSize (mhaRunner.cu:522-525)
    size_t unfusedWorkspace(DataType type, int32_t numHeads) const
    {
        return setUp ? trtamd_unfused_mha_workspace_size(static_cast<int32_t>(type), S, B, numHeads) : 0;
    }
};

// Is there a fused fixed-length (packed-mask) kernel for this type, head size and S?  The reference
// has them for S in {64,96,128,384} (FP16) and {128,384} (INT8), the sizes for which the
// embedding plugin emits a packed mask (mhaRunner.cu:676-692, 805-821).
bool fusedV1Valid(DataType type, int32_t headSize, int32_t S)
{
    if (headSize != 64)
    {
        return false;
    }
    if (type == DataType::kHALF)
    {
        return S == 64 || S == 96 || S == 128 || S == 384;
    }
    if (type == DataType::kINT8)
    {
        return S == 128 || S == 384;
    }
    return false;
}

// What creating a fused runner does in the reference (getXMMAKernels / getXMMAKernelsV2 load every kernel and raise
// its shared-memory limit, fused_multihead_attention.h:63-147): afterwards enqueue only launches.  Only the types the
// fused kernels serve ask for it, and a failure is logged, not thrown: a launch raises the limit of its own kernel
// again if it has to, and an object that never launches a fused kernel must not fail to exist over them.
void prepareFusedKernels(DataType type)
{
    if ((type == DataType::kHALF || type == DataType::kINT8) && deviceAvailable()
        && trtamd_fused_mha_prepare() != TRTAMD_STATUS_SUCCESS)
    {
        logMessage(ILogger::Severity::kWARNING,
            std::string("fused attention kernels could not be prepared ahead of the first enqueue: ") + trtamd_last_error());
    }
}

void fillInt8Scales(trtamd_fmha_params& p, float scaleQkv, float scaleCtx, float rsqrtHeadSize, float dqProbs)
{
    // FusedMHARunnerInt8{,v2}::mhaImpl::run (mhaRunner.cu:838-850, 1178-1190)
    float const scaleBmm1 = scaleQkv * scaleQkv * rsqrtHeadSize;
    float const scaleBmm2 = dqProbs * scaleQkv / scaleCtx;
    float const scaleSoftmax = 1.F / dqProbs;
    p.scale_bmm1 = floatBits(scaleBmm1);
    p.scale_bmm2 = floatBits(scaleBmm2);
    p.scale_softmax = floatBits(scaleSoftmax);
    p.enable_i2f_trick
        = -double(1 << 22) * double(scaleBmm2) <= -128.F && double(1 << 22) * double(scaleBmm2) >= 127.F;
}

void fillFp16Scales(trtamd_fmha_params& p, float rsqrtHeadSize)
{
    // set_alpha with DATA_TYPE_FP16 (mhaRunner.cu:608-628, 694-701)
    p.scale_bmm1 = half2Bits(rsqrtHeadSize);
    p.scale_softmax = half2Bits(1.F);
    p.scale_bmm2 = half2Bits(1.F);
}

int32_t runUnfused(DataType type, RunnerState const& st, int32_t numHeads, void const* qkv, void const* maskIdx,
    void* output, void* workspace, hipStream_t stream)
{
    TRTAMD_VALIDATE_MSG(type != DataType::kINT8, "The Unfused MHARunner does not support INT8!");
    TRTAMD_VALIDATE(workspace != nullptr);
    checkKernelStatus(trtamd_unfused_mha_routed(stream, st.route(), static_cast<int32_t>(type), st.S, st.B, numHeads,
                          st.headSize, qkv, static_cast<int32_t const*>(maskIdx), output, workspace),
        "unfused attention");
    return 0;
}

// ------------------------------------------------------------------------------------------
// version 4
// ------------------------------------------------------------------------------------------
class QkvToContextPlugin final : public BertPluginBase
{
public:
    // build-phase constructor
    QkvToContextPlugin(std::string const& name, DataType type, int32_t hiddenSize, int32_t numHeads, float dqProbs,
        bool hasMask)
        : BertPluginBase(name, kNAME, "4", 1 + (hasMask ? 1 : 0), 1)
        , mHeadSize(hiddenSize / numHeads)
        , mHiddenSize(hiddenSize)
        , mNumHeads(numHeads)
        , mType(type)
        , mDqProbs(dqProbs)
        , mHasMask(hasMask ? 1 : 0)
    {
        mSM = getSmVersion();
        mUnfused.unfused = true;
        prepareFusedKernels(mType);
    }

    // runtime-phase constructor (deserialised engine)
    QkvToContextPlugin(std::string const& name, DataType type, int32_t S, int32_t B, int32_t SM, int32_t hiddenSize,
        int32_t numHeads, float dqProbs, bool hasMask, bool hasUnfusedDispatcher, void const* runnerState,
        int64_t runnerStateBytes = -1)
        : QkvToContextPlugin(name, type, hiddenSize, numHeads, dqProbs, hasMask)
    {
        mS = S;
        mB = B;
        mSM = SM;
        if (hasUnfusedDispatcher)
        {
            TRTAMD_VALIDATE(runnerState != nullptr);
            mUnfused.deserialize(runnerState, runnerStateBytes);
        }
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        std::vector<uint8_t> buf;
        bool const has = mUnfused.unfusedWorkspace(mType, mNumHeads) != 0;
        if (has)
        {
            mUnfused.serialize(buf);
        }
        return std::make_unique<QkvToContextPlugin>(mLayerName, mType, mS, mB, mSM, mHiddenSize, mNumHeads, mDqProbs,
            mHasMask != 0, has, has ? buf.data() : nullptr);
    }

    void doOutputTypes(DataType* outputTypes, DataType const* inputTypes) const override
    {
        TRTAMD_VALIDATE(inputTypes[0] == DataType::kFLOAT || inputTypes[0] == DataType::kHALF
            || inputTypes[0] == DataType::kINT8);
        outputTypes[0] = inputTypes[0];
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) override
    {
        // [S,B,3E,1,1] -> [S,B,E,1,1]
        outputs[0] = inputs[kIIDX];
        outputs[0].d[kHDIM] = eb.operation(DimensionOperation::kFLOOR_DIV, *inputs[kIIDX].d[kHDIM], *eb.constant(3));
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        auto const* in = inOut;
        auto const* out = inOut + expectedInputs();
        int32_t const packedSize = getMHAMaskPackedSize(mSM, mType, static_cast<int32_t>(in->desc.dims.d[kSDIM]));
        if (mType == DataType::kINT8)
        {
            // INT8 has no unfused fallback: the sequence length must be static and have a packed mask
            if (in->desc.dims.d[kSDIM] == -1)
            {
                logMessage(ILogger::Severity::kERROR,
                    std::string("INT8 IO not support dynamic shape in sequence dimension for plugin ") + kNAME);
                return false;
            }
            if (packedSize == kUnfusedMaskSize)
            {
                logMessage(ILogger::Severity::kERROR,
                    std::string("INT8 IO only support sequence length 128,384 for plugin ") + kNAME);
                return false;
            }
        }
        auto int8Format = [](int64_t hidden) { return hidden % 32 == 0 ? TensorFormat::kCHW32 : TensorFormat::kCHW4; };
        if (pos == 0)
        {
            TensorFormat const want = mType == DataType::kINT8 ? int8Format(in->desc.dims.d[kHDIM]) : TensorFormat::kLINEAR;
            return in->desc.type == mType && in->desc.format == want && in->desc.dims.nbDims == 5
                && in->desc.dims.d[kHDIM] % 3 == 0 && in->desc.dims.d[3] == 1 && in->desc.dims.d[4] == 1;
        }
        if (mHasMask && pos == 1)
        {
            PluginTensorDesc const& mask = inOut[1].desc;
            if (mask.dims.d[1] != -1 && mask.dims.d[1] != packedSize)
            {
                logMessage(ILogger::Severity::kERROR,
                    "CustomEmbLayerNormPluginDynamic returned mask with pack size " + std::to_string(mask.dims.d[1])
                        + ", but " + kNAME + " expects mask pack size " + std::to_string(packedSize));
                return false;
            }
            return mask.type == DataType::kINT32 && mask.format == TensorFormat::kLINEAR && mask.dims.nbDims == 2
                && mask.dims.d[0] == in->desc.dims.d[kBDIM];
        }
        if (!mHasMask || pos == 2)
        {
            TensorFormat const want
                = mType == DataType::kINT8 ? int8Format(out->desc.dims.d[kHDIM]) : TensorFormat::kLINEAR;
            return in->desc.type == out->desc.type && out->desc.format == want && out->desc.dims.nbDims == 5
                && in->desc.dims.d[kHDIM] / 3 == out->desc.dims.d[kHDIM] && out->desc.dims.d[3] == 1
                && out->desc.dims.d[4] == 1 && out->desc.dims.d[kBDIM] == in->desc.dims.d[kBDIM]
                && out->desc.dims.d[kSDIM] == in->desc.dims.d[kSDIM];
        }
        return false;
    }

    void checkDescs(PluginTensorDesc const& inDesc, PluginTensorDesc const& outDesc, PluginTensorDesc const* maskDesc)
    {
        TRTAMD_VALIDATE(mType == inDesc.type);
        TRTAMD_VALIDATE(mType == outDesc.type);
        TRTAMD_VALIDATE(inDesc.dims.d[kBDIM] == outDesc.dims.d[kBDIM]);
        TRTAMD_VALIDATE(inDesc.dims.d[kSDIM] == outDesc.dims.d[kSDIM]);
        TRTAMD_VALIDATE(inDesc.dims.d[kHDIM] == 3 * outDesc.dims.d[kHDIM]);
        if (maskDesc)
        {
            TRTAMD_VALIDATE(maskDesc->dims.d[0] == inDesc.dims.d[kBDIM]);
        }
    }

    void doConfigure(DynamicPluginTensorDesc const* in, DynamicPluginTensorDesc const* out) override
    {
        PluginTensorDesc const& inDesc = in[kIIDX].desc;
        checkDescs(inDesc, out->desc, mHasMask ? &in[kMIDX].desc : nullptr);
        int32_t const S = static_cast<int32_t>(inDesc.dims.d[kSDIM]);
        int32_t const B = static_cast<int32_t>(inDesc.dims.d[kBDIM] <= 0 ? in->max.d[kBDIM] : inDesc.dims.d[kBDIM]);
        bool const hasFused = mType == DataType::kHALF || mType == DataType::kINT8;
        if (S <= 0)
        {
            // dynamic sequence length: size the workspace for the longest length that cannot be fused
            int32_t const smin = static_cast<int32_t>(in->min.d[kSDIM]);
            int32_t const smax = static_cast<int32_t>(in->max.d[kSDIM]);
            if (hasFused)
            {
                for (int32_t i = smax; i >= smin; --i)
                {
                    if (!fusedV1Valid(mType, mHeadSize, i))
                    {
                        mUnfused.setup(i, B, mHeadSize);
                        mS = i;
                        mB = B;
                        break;
                    }
                }
            }
            else
            {
                mUnfused.setup(smax, B, mHeadSize);
                mS = smax;
                mB = B;
            }
        }
        else
        {
            if (!(hasFused && fusedV1Valid(mType, mHeadSize, S)))
            {
                mUnfused.setup(S, B, mHeadSize);
            }
            mS = S;
            mB = B;
        }
        mUnfused.tune(mType, mNumHeads);
    }

    size_t doWorkspaceSize(DynamicPluginTensorDesc const*, DynamicPluginTensorDesc const*) const override
    {
        // only the unfused path needs scratch, sized by the set-up done in configurePlugin
        return mUnfused.unfusedWorkspace(mType, mNumHeads);
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const* out) override
    {
        PluginTensorDesc const& inDesc = in[kIIDX];
        checkDescs(inDesc, out[0], mHasMask ? &in[kMIDX] : nullptr);
        mS = static_cast<int32_t>(inDesc.dims.d[kSDIM]);
        mB = static_cast<int32_t>(inDesc.dims.d[kBDIM]);
        TRTAMD_VALIDATE(mS);
        TRTAMD_VALIDATE(mB);
        if (!fusedV1Valid(mType, mHeadSize, mS))
        {
            mUnfused.setup(mS, mB, mHeadSize);
        }
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void* workspace, hipStream_t stream) override
    {
        TRTAMD_VALIDATE(mS == inputDesc->dims.d[kSDIM]);
        TRTAMD_VALIDATE(mB == inputDesc->dims.d[kBDIM]);
        void const* maskPtr = mHasMask ? inputs[1] : nullptr;
        if (mHasMask && fusedV1Valid(mType, mHeadSize, mS))
        {
            // FusedMHARunner{FP16,Int8}: fixed layout, packed mask (mhaRunner.cu:630-918)
            trtamd_fmha_params p{};
            int64_t const esize = getElementSize(mType);
            p.qkv_ptr = inputs[0];
            p.packed_mask_ptr = maskPtr;
            p.o_ptr = outputs[0];
            p.b = mB;
            p.h = mNumHeads;
            p.s = mS;
            p.d = mHeadSize;
            p.qkv_stride_in_bytes = int64_t(3) * mB * mNumHeads * mHeadSize * esize; // mLdQKV
            p.o_stride_in_bytes = int64_t(mB) * mNumHeads * mHeadSize * esize;       // mLdOut
            // The embedding plugin sizes the mask tensor for S = 128 but packs S = 64 and 96 densely:
            // the per-sequence stride is xmmas_m * threads words (mhaRunner.cu:676-697, 818-831)
            int32_t const warpsM = mS == 384 ? 1 : 2;
            int32_t const threads = mS == 384 ? 256 : 128;
            int32_t const xmmasM = (mS + 16 * warpsM - 1) / (16 * warpsM);
            p.packed_mask_stride_in_bytes = int64_t(xmmasM) * threads * 4;
            float const rsqrtHead = 1.F / std::sqrt(static_cast<float>(mHeadSize));
            if (mType == DataType::kINT8)
            {
                fillInt8Scales(p, inputDesc[0].scale, outputDesc[0].scale, rsqrtHead, mDqProbs);
            }
            else
            {
                fillFp16Scales(p, rsqrtHead);
            }
            checkKernelStatus(trtamd_fused_mha_run(stream, static_cast<int32_t>(mType), &p), "fused attention");
            return 0;
        }
        RunnerState st = mUnfused;
        if (!st.setUp)
        {
            st.setup(mS, mB, mHeadSize);
        }
        return runUnfused(mType, st, mNumHeads, inputs[0], maskPtr, outputs[0], workspace, stream);
    }

    void doSerialize(FieldList& f) override
    {
        f.add("type_id", &mType, PluginFieldType::kINT32, 1);
        f.add("hidden_size", &mHiddenSize, PluginFieldType::kINT32, 1);
        f.add("num_heads", &mNumHeads, PluginFieldType::kINT32, 1);
        f.add("has_mask", &mHasMask, PluginFieldType::kINT32, 1);
        f.add("S", &mS, PluginFieldType::kINT32, 1);
        f.add("B", &mB, PluginFieldType::kINT32, 1);
        f.add("SM", &mSM, PluginFieldType::kINT32, 1);
        if (mUnfused.unfusedWorkspace(mType, mNumHeads) != 0)
        {
            mHasUnfusedDispatcher = 1;
            mUnfused.serialize(mRunnerStateBuffer);
            f.add("runnerStateBuffer", mRunnerStateBuffer.data(), PluginFieldType::kUNKNOWN,
                static_cast<int32_t>(mRunnerStateBuffer.size()));
        }
        else
        {
            mHasUnfusedDispatcher = 0;
        }
        f.add("hasUnfusedDispatcher", &mHasUnfusedDispatcher, PluginFieldType::kINT32, 1);
        if (mDqProbs >= 0)
        {
            f.add("dq_probs", &mDqProbs, PluginFieldType::kFLOAT32, 1);
        }
    }

private:
    int32_t mS{0};
    int32_t mB{0};
    int32_t mSM{0};
    int32_t mHeadSize;
    int32_t mHiddenSize;
    int32_t mNumHeads;
    DataType mType;
    float mDqProbs;
    int32_t mHasMask;
    int32_t mHasUnfusedDispatcher{0};
    RunnerState mUnfused;
    std::vector<uint8_t> mRunnerStateBuffer;
};

// shared parsing of the attributes versions 4 and 5 have in common
struct QkvCommonFields
{
    int32_t typeId{-1};
    int32_t hiddenSize{0};
    int32_t numHeads{-1};
    bool hasMask{false};
    float dqProbs{-1.F};
    int32_t s{-1}, b{-1};
    void const* runnerState{nullptr};
    int64_t runnerStateBytes{-1};

    void read(PluginFieldCollection const* fc, TensorRTPhase phase)
    {
        for (int32_t i = 0; i < fc->nbFields; ++i)
        {
            TRTAMD_VALIDATE(fc->fields[i].data != nullptr);
        }
        if (readScalar(fc, "type_id", typeId))
        {
            TRTAMD_VALIDATE_MSG(typeId >= 0 && typeId <= 2, "QKV: Invalid TypeId " + std::to_string(typeId));
        }
        if (readScalar(fc, "hidden_size", hiddenSize))
        {
            TRTAMD_VALIDATE_MSG(hiddenSize > 0, "QKV: Invalid hiddenSize " + std::to_string(hiddenSize));
        }
        if (readScalar(fc, "num_heads", numHeads))
        {
            TRTAMD_VALIDATE_MSG(numHeads > 0, "QKV: Invalid numHeads " + std::to_string(numHeads));
        }
        int32_t hasMaskValue = 0;
        if (readScalar(fc, "has_mask", hasMaskValue))
        {
            TRTAMD_VALIDATE_MSG(
                hasMaskValue == 0 || hasMaskValue == 1, "QKV: Invalid hasMask " + std::to_string(hasMaskValue));
            hasMask = hasMaskValue != 0;
        }
        if (readScalar(fc, "dq_probs", dqProbs))
        {
            TRTAMD_VALIDATE_MSG(dqProbs > 0.0F, "QKV: Invalid dqProbs " + std::to_string(dqProbs));
        }
        bool const runtimeOnly = findField(fc, "S") || findField(fc, "B") || findField(fc, "runnerStateBuffer");
        TRTAMD_VALIDATE_MSG(!runtimeOnly || phase == TensorRTPhase::kRUNTIME,
            "S, B and runnerStateBuffer are runtime-phase fields");
        readScalar(fc, "S", s);
        readScalar(fc, "B", b);
        if (PluginField const* f = findField(fc, "runnerStateBuffer"))
        {
            runnerState = f->data;
            runnerStateBytes = f->length;
        }
        if (static_cast<DataType>(typeId) == DataType::kINT8 && dqProbs < 0)
        {
            dqProbs = 1.F / 127.F;
        }
    }
};

class QkvToContextCreator final : public BertCreatorBase
{
public:
    QkvToContextCreator()
        : BertCreatorBase(kNAME, "4",
            {PluginField("type_id", nullptr, PluginFieldType::kINT32, 1),
                PluginField("hidden_size", nullptr, PluginFieldType::kINT32, 1),
                PluginField("num_heads", nullptr, PluginFieldType::kINT32, 1),
                PluginField("has_mask", nullptr, PluginFieldType::kINT32, 1),
                PluginField("dq_probs", nullptr, PluginFieldType::kFLOAT32, 1)})
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc,
        TensorRTPhase phase) override
    {
        if (phase == TensorRTPhase::kBUILD)
        {
            validateRequiredFields({"type_id", "hidden_size", "num_heads", "has_mask"}, fc);
        }
        else
        {
            validateRequiredFields(
                {"type_id", "S", "B", "hidden_size", "num_heads", "has_mask", "SM", "hasUnfusedDispatcher"}, fc);
        }
        QkvCommonFields c;
        c.read(fc, phase);
        int32_t sm = -1;
        int32_t hasUnfused = 0;
        TRTAMD_VALIDATE_MSG(phase == TensorRTPhase::kRUNTIME || (!findField(fc, "SM") && !findField(fc, "hasUnfusedDispatcher")),
            "SM and hasUnfusedDispatcher are runtime-phase fields");
        readScalar(fc, "SM", sm);
        if (readScalar(fc, "hasUnfusedDispatcher", hasUnfused))
        {
            TRTAMD_VALIDATE_MSG(hasUnfused == 0 || hasUnfused == 1,
                "QKV: Invalid hasUnfusedDispatcher " + std::to_string(hasUnfused));
        }
        auto const type = static_cast<DataType>(c.typeId);
        if (phase == TensorRTPhase::kBUILD)
        {
            return std::make_unique<QkvToContextPlugin>(name, type, c.hiddenSize, c.numHeads, c.dqProbs, c.hasMask);
        }
        TRTAMD_VALIDATE_MSG(c.s != -1, "invalid S during runtime plugin creation");
        TRTAMD_VALIDATE_MSG(c.b != -1, "invalid B during runtime plugin creation");
        TRTAMD_VALIDATE_MSG(sm != -1, "invalid SM during runtime plugin creation");
        if (hasUnfused == 1)
        {
            TRTAMD_VALIDATE_MSG(c.runnerState != nullptr, "invalid runnerStateBuffer during runtime plugin creation");
        }
        else
        {
            TRTAMD_VALIDATE_MSG(c.runnerState == nullptr, "invalid runnerStateBuffer during runtime plugin creation");
        }
        return std::make_unique<QkvToContextPlugin>(name, type, c.s, c.b, sm, c.hiddenSize, c.numHeads, c.dqProbs,
            c.hasMask, hasUnfused == 1, c.runnerState, c.runnerStateBytes);
    }
};

// ------------------------------------------------------------------------------------------
// version 5
// ------------------------------------------------------------------------------------------
class QkvToContextVarSeqlenPlugin final : public BertPluginBase
{
public:
    QkvToContextVarSeqlenPlugin(std::string const& name, DataType type, int32_t hiddenSize, int32_t numHeads,
        float dqProbs, bool hasMask, bool varSeqlen, bool useInt8ScaleMax)
        : BertPluginBase(name, kNAME, "5", 1 + (hasMask ? 1 : 0) + (varSeqlen ? 2 : 0), 1)
        , mHeadSize(hiddenSize / numHeads)
        , mHiddenSize(hiddenSize)
        , mNumHeads(numHeads)
        , mType(type)
        , mDqProbs(dqProbs)
        , mHasMask(hasMask ? 1 : 0)
        , mUseVarSeqlen(varSeqlen ? 1 : 0)
        , mUseInt8ScaleMax(useInt8ScaleMax ? 1 : 0)
        , mHdim(varSeqlen ? 1 : kHDIM)
    {
        mSM = getSmVersion();
        if (varSeqlen)
        {
            // variable sequence length exists for the fused kernels only; the packed layout puts the
            // hidden dimension second: [T, 3E, 1, 1]
            TRTAMD_VALIDATE_MSG(type == DataType::kINT8 || type == DataType::kHALF,
                "requesting maxSeqlen not compatible with GPU arch");
            TRTAMD_VALIDATE(mHeadSize <= 64);
        }
        else
        {
            TRTAMD_VALIDATE(mType != DataType::kINT8);
        }
        mRunner.unfused = !varSeqlen;
        prepareFusedKernels(mType);
    }

    QkvToContextVarSeqlenPlugin(std::string const& name, int32_t S, int32_t B, DataType type, int32_t hiddenSize,
        int32_t numHeads, float dqProbs, bool hasMask, bool varSeqlen, bool useInt8ScaleMax, void const* runnerState,
        int64_t runnerStateBytes = -1)
        : QkvToContextVarSeqlenPlugin(name, type, hiddenSize, numHeads, dqProbs, hasMask, varSeqlen, useInt8ScaleMax)
    {
        mS = S;
        mB = B;
        TRTAMD_VALIDATE(runnerState != nullptr);
        mRunner.deserialize(runnerState, runnerStateBytes);
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        if (mRunner.setUp)
        {
            std::vector<uint8_t> buf;
            mRunner.serialize(buf);
            return std::make_unique<QkvToContextVarSeqlenPlugin>(mLayerName, mS, mB, mType, mHiddenSize, mNumHeads,
                mDqProbs, mHasMask != 0, mUseVarSeqlen != 0, mUseInt8ScaleMax != 0, buf.data());
        }
        return std::make_unique<QkvToContextVarSeqlenPlugin>(mLayerName, mType, mHiddenSize, mNumHeads, mDqProbs,
            mHasMask != 0, mUseVarSeqlen != 0, mUseInt8ScaleMax != 0);
    }

    void doOutputTypes(DataType* outputTypes, DataType const* inputTypes) const override
    {
        TRTAMD_VALIDATE(inputTypes[0] == DataType::kFLOAT || inputTypes[0] == DataType::kHALF
            || inputTypes[0] == DataType::kINT8);
        outputTypes[0] = inputTypes[0];
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) override
    {
        outputs[0] = inputs[kIIDX];
        outputs[0].d[mHdim] = eb.operation(DimensionOperation::kFLOOR_DIV, *inputs[kIIDX].d[mHdim], *eb.constant(3));
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        int32_t const nbInputs = expectedInputs();
        auto const* in = inOut;
        auto const* out = inOut + nbInputs;
        if (mUseVarSeqlen)
        {
            TRTAMD_VALIDATE_MSG(nbInputs == 4, "for varseqlen, expected 4 inputs");
        }
        Dims const& inDims = in->desc.dims;
        Dims const& outDims = out->desc.dims;
        TensorFormat supportedFormat = TensorFormat::kLINEAR;
        if (mType == DataType::kINT8)
        {
            supportedFormat = inDims.d[mHdim] % 32 == 0 ? TensorFormat::kCHW32 : TensorFormat::kCHW4;
        }
        int32_t const supportedNbDims = mUseVarSeqlen ? 4 : 5;
        bool const supportedHdim = pos == 0 ? inDims.d[mHdim] % 3 == 0 : inDims.d[mHdim] / 3 == outDims.d[mHdim];
        if (pos == 0 || pos == nbInputs)
        {
            PluginTensorDesc const& desc = inOut[pos].desc;
            return desc.type == mType && desc.format == supportedFormat && desc.dims.nbDims == supportedNbDims
                && supportedHdim && desc.dims.d[mHdim + 1] == 1 && desc.dims.d[mHdim + 2] == 1;
        }
        TRTAMD_VALIDATE(mHasMask);
        if (pos == 1)
        {
            if (mUseVarSeqlen)
            {
                return true; // dummy input
            }
            PluginTensorDesc const& mask = inOut[pos].desc;
            return mask.format == TensorFormat::kLINEAR && mask.type == DataType::kINT32 && mask.dims.nbDims == 1;
        }
        TRTAMD_VALIDATE(mUseVarSeqlen);
        if (pos == 2)
        {
            PluginTensorDesc const& seqlens = inOut[pos].desc;
            return seqlens.type == DataType::kINT32 && seqlens.format == TensorFormat::kLINEAR;
        }
        if (pos == 3)
        {
            return inOut[pos].desc.dims.nbDims == 1;
        }
        return false;
    }

    void checkFixedDescs(PluginTensorDesc const& inDesc, PluginTensorDesc const& outDesc, PluginTensorDesc const* mask)
    {
        TRTAMD_VALIDATE(inDesc.dims.d[kBDIM] == outDesc.dims.d[kBDIM]);
        TRTAMD_VALIDATE(inDesc.dims.d[kSDIM] == outDesc.dims.d[kSDIM]);
        TRTAMD_VALIDATE(inDesc.dims.d[mHdim] == 3 * outDesc.dims.d[mHdim]);
        if (mask)
        {
            TRTAMD_VALIDATE(mask->dims.d[0] == inDesc.dims.d[kBDIM]);
        }
    }

    void doConfigure(DynamicPluginTensorDesc const* in, DynamicPluginTensorDesc const* out) override
    {
        PluginTensorDesc const& inDesc = in[kIIDX].desc;
        TRTAMD_VALIDATE(mType == inDesc.type);
        TRTAMD_VALIDATE(mType == out->desc.type);
        if (!mUseVarSeqlen)
        {
            checkFixedDescs(inDesc, out->desc, mHasMask ? &in[kMIDX].desc : nullptr);
            int32_t const S
                = static_cast<int32_t>(inDesc.dims.d[kSDIM] <= 0 ? in->max.d[kSDIM] : inDesc.dims.d[kSDIM]);
            int32_t const B
                = static_cast<int32_t>(inDesc.dims.d[kBDIM] <= 0 ? in->max.d[kBDIM] : inDesc.dims.d[kBDIM]);
            if (S != mS || B != mB)
            {
                mRunner.setup(S, B, mHeadSize);
                mS = S;
                mB = B;
            }
            mRunner.tune(mType, mNumHeads);
        }
        else
        {
            // placeholder geometry; the real batch and bucket are set at enqueue
            mRunner.setup(256, 1, mHeadSize);
        }
    }

    size_t doWorkspaceSize(DynamicPluginTensorDesc const* inputs, DynamicPluginTensorDesc const*) const override
    {
        size_t padding = 0;
        if (mUseVarSeqlen && mHeadSize != 64)
        {
            // QkvPaddingRunner::getWorkspaceSize (zeroPadding2d.cu:167-171): padded QKV + padded
            // output at head size 64 + 16 bytes of alignment slack
            size_t const esize = getElementSize(mType);
            size_t const sumSeqLen = static_cast<size_t>(inputs[0].desc.dims.d[0] < 0 ? inputs[0].max.d[0] : inputs[0].desc.dims.d[0]);
            padding = 4U * sumSeqLen * mNumHeads * 64U * esize + 16U;
        }
        size_t const runner = mRunner.unfused ? mRunner.unfusedWorkspace(mType, mNumHeads) : 0;
        return runner + padding;
    }

    void doShapeChange(PluginTensorDesc const* in, PluginTensorDesc const* out) override
    {
        TRTAMD_VALIDATE(mType == in[kIIDX].type);
        TRTAMD_VALIDATE(mType == out[0].type);
        if (!mUseVarSeqlen)
        {
            checkFixedDescs(in[kIIDX], out[0], mHasMask ? &in[kMIDX] : nullptr);
            // configurePlugin (build) or the deserialised fields (runtime) provided S and B
            TRTAMD_VALIDATE(mS);
            TRTAMD_VALIDATE(mB);
            mRunner.setup(mS, mB, mHeadSize);
        }
        else
        {
            mRunner.setup(256, 1, mHeadSize);
        }
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void* workspace, hipStream_t stream) override
    {
        if (!mUseVarSeqlen)
        {
            TRTAMD_VALIDATE(mS == inputDesc->dims.d[kSDIM]);
            TRTAMD_VALIDATE(mB == inputDesc->dims.d[kBDIM]);
            void const* maskPtr = mHasMask ? inputs[1] : nullptr;
            RunnerState st = mRunner;
            if (!st.setUp)
            {
                st.setup(mS, mB, mHeadSize);
            }
            return runUnfused(mType, st, mNumHeads, inputs[0], maskPtr, outputs[0], workspace, stream);
        }
        int32_t const B = static_cast<int32_t>(inputDesc[2].dims.d[0]) - 1;
        int32_t const maxS = static_cast<int32_t>(inputDesc[3].dims.d[0]);
        TRTAMD_VALIDATE_MSG(maxS <= 512,
            "No implementation for variable sequence length multi-head attention plugin with sequence > 512.");
        // kernel bucket of the reference (qkvToContextPlugin.cpp:1223-1251); results depend on
        // cu_seqlens only, the bucket merely bounds the per-sequence capacity
        int32_t S = 512;
        if (mType == DataType::kHALF && maxS <= 64)
        {
            S = 64;
        }
        else if (mType == DataType::kHALF && maxS <= 96)
        {
            S = 96;
        }
        else if (maxS <= 128)
        {
            S = 128;
        }
        else if (maxS <= 192)
        {
            S = mType == DataType::kHALF ? 256 : 192;
        }
        else if (maxS <= 256)
        {
            S = 256;
        }
        else if (maxS <= 384)
        {
            S = 384;
        }
        // head sizes below 64 are zero-padded: to 32 when they fit, else to 64; the softmax scale
        // follows the padded size, as in the reference (runV2Kernel sets the runner up with padSize)
        int32_t const padSize = mHeadSize <= 32 ? 32 : 64;
        mRunner.setup(S, B, padSize);
        int64_t const esize = getElementSize(mType);
        int64_t const sumSeqLen = inputDesc[0].dims.d[0];
        void const* qkv = inputs[0];
        void* ctx = outputs[0];
        void* paddedOut = nullptr;
        constexpr int32_t kKernelHead = 64; // the fused kernels of this library exist for head size 64
        if (mHeadSize != kKernelHead)
        {
            TRTAMD_VALIDATE(workspace != nullptr);
            auto addr = reinterpret_cast<uintptr_t>(workspace);
            addr = (addr + 15) & ~uintptr_t(15);
            void* paddedIn = reinterpret_cast<void*>(addr);
            size_t const inBytes = static_cast<size_t>(3 * sumSeqLen * mNumHeads * kKernelHead * esize);
            paddedOut = reinterpret_cast<void*>((addr + inBytes + 15) & ~uintptr_t(15));
            checkKernelStatus(trtamd_zero_padding_2d(inputs[0], static_cast<int32_t>(mHeadSize * esize), paddedIn,
                                  static_cast<int32_t>(kKernelHead * esize),
                                  static_cast<int32_t>(3 * sumSeqLen * mNumHeads), stream),
                "head-size padding");
            qkv = paddedIn;
            ctx = paddedOut;
        }
        trtamd_fmha_params p{};
        p.qkv_ptr = qkv;
        p.o_ptr = ctx;
        p.cu_seqlens = static_cast<int32_t const*>(inputs[2]);
        p.b = B;
        p.h = mNumHeads;
        p.s = S;
        p.d = kKernelHead;
        p.qkv_stride_in_bytes = int64_t(3) * mNumHeads * kKernelHead * esize;
        p.o_stride_in_bytes = int64_t(mNumHeads) * kKernelHead * esize;
        p.use_int8_scale_max = mUseInt8ScaleMax;
        float const rsqrtHead = 1.F / std::sqrt(static_cast<float>(padSize));
        if (mType == DataType::kINT8)
        {
            fillInt8Scales(p, inputDesc[0].scale, outputDesc[0].scale, rsqrtHead, mDqProbs);
        }
        else
        {
            fillFp16Scales(p, rsqrtHead);
        }
        checkKernelStatus(trtamd_fused_mha_run(stream, static_cast<int32_t>(mType), &p), "fused attention");
        if (paddedOut)
        {
            checkKernelStatus(trtamd_zero_padding_2d(paddedOut, static_cast<int32_t>(kKernelHead * esize), outputs[0],
                                  static_cast<int32_t>(mHeadSize * esize),
                                  static_cast<int32_t>(sumSeqLen * mNumHeads), stream),
                "head-size unpadding");
        }
        return 0;
    }

    void doSerialize(FieldList& f) override
    {
        f.add("type_id", &mType, PluginFieldType::kINT32, 1);
        f.add("hidden_size", &mHiddenSize, PluginFieldType::kINT32, 1);
        f.add("num_heads", &mNumHeads, PluginFieldType::kINT32, 1);
        f.add("has_mask", &mHasMask, PluginFieldType::kINT32, 1);
        f.add("var_seqlen", &mUseVarSeqlen, PluginFieldType::kINT32, 1);
        f.add("use_int8_scale_max", &mUseInt8ScaleMax, PluginFieldType::kINT32, 1);
        f.add("S", &mS, PluginFieldType::kINT32, 1);
        f.add("B", &mB, PluginFieldType::kINT32, 1);
        mRunner.serialize(mRunnerStateBuffer);
        f.add("runnerStateBuffer", mRunnerStateBuffer.data(), PluginFieldType::kUNKNOWN,
            static_cast<int32_t>(mRunnerStateBuffer.size()));
        if (mDqProbs >= 0)
        {
            f.add("dq_probs", &mDqProbs, PluginFieldType::kFLOAT32, 1);
        }
    }

private:
    int32_t mS{0};
    int32_t mB{0};
    int32_t mSM{0};
    int32_t mHeadSize;
    int32_t mHiddenSize;
    int32_t mNumHeads;
    DataType mType;
    float mDqProbs;
    int32_t mHasMask;
    int32_t mUseVarSeqlen;
    int32_t mUseInt8ScaleMax;
    int32_t mHdim;
    RunnerState mRunner;
    std::vector<uint8_t> mRunnerStateBuffer;
};

class QkvToContextVarSeqlenCreator final : public BertCreatorBase
{
public:
    QkvToContextVarSeqlenCreator()
        : BertCreatorBase(kNAME, "5",
            {PluginField("type_id", nullptr, PluginFieldType::kINT32, 1),
                PluginField("hidden_size", nullptr, PluginFieldType::kINT32, 1),
                PluginField("num_heads", nullptr, PluginFieldType::kINT32, 1),
                PluginField("has_mask", nullptr, PluginFieldType::kINT32, 1),
                PluginField("dq_probs", nullptr, PluginFieldType::kFLOAT32, 1),
                PluginField("var_seqlen", nullptr, PluginFieldType::kINT32, 1),
                PluginField("use_int8_scale_max", nullptr, PluginFieldType::kINT32, 1)})
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc,
        TensorRTPhase phase) override
    {
        if (phase == TensorRTPhase::kBUILD)
        {
            validateRequiredFields({"type_id", "hidden_size", "num_heads", "has_mask"}, fc);
        }
        else
        {
            validateRequiredFields({"type_id", "S", "B", "hidden_size", "num_heads", "has_mask", "var_seqlen",
                                       "use_int8_scale_max", "runnerStateBuffer"},
                fc);
        }
        QkvCommonFields c;
        c.read(fc, phase);
        int32_t varSeqlen = 0;
        int32_t useInt8ScaleMax = -1;
        readScalar(fc, "var_seqlen", varSeqlen);
        if (readScalar(fc, "use_int8_scale_max", useInt8ScaleMax))
        {
            TRTAMD_VALIDATE_MSG(useInt8ScaleMax == 0 || useInt8ScaleMax == 1,
                "QKV: Invalid useInt8ScaleMax " + std::to_string(useInt8ScaleMax));
        }
        if (useInt8ScaleMax < 0)
        {
            logMessage(ILogger::Severity::kINFO, "Using default for use_int8_scale_max: true");
            useInt8ScaleMax = 1;
        }
        auto const type = static_cast<DataType>(c.typeId);
        if (phase == TensorRTPhase::kBUILD)
        {
            return std::make_unique<QkvToContextVarSeqlenPlugin>(name, type, c.hiddenSize, c.numHeads, c.dqProbs,
                c.hasMask, varSeqlen != 0, useInt8ScaleMax != 0);
        }
        TRTAMD_VALIDATE_MSG(c.s != -1, "invalid S during runtime plugin creation");
        TRTAMD_VALIDATE_MSG(c.b != -1, "invalid B during runtime plugin creation");
        TRTAMD_VALIDATE_MSG(c.runnerState != nullptr, "invalid runnerStateBuffer during runtime plugin creation");
        return std::make_unique<QkvToContextVarSeqlenPlugin>(name, c.s, c.b, type, c.hiddenSize, c.numHeads, c.dqProbs,
            c.hasMask, varSeqlen != 0, useInt8ScaleMax != 0, c.runnerState, c.runnerStateBytes);
    }
};

// ------------------------------------------------------------------------------------------
// version 6
// ------------------------------------------------------------------------------------------
class QkvToContextInterleavedPlugin final : public BertPluginBase
{
public:
    QkvToContextInterleavedPlugin(std::string const& name, int32_t hiddenSize, int32_t numHeads, float dqProbs,
        bool useInt8ScaleMax, bool useExplicitInt8, float qkvScale, float ctxScale)
        : BertPluginBase(name, kNAME, "6", 3, 1)
        , mHeadSize(hiddenSize / numHeads)
        , mHiddenSize(hiddenSize)
        , mNumHeads(numHeads)
        , mDqProbs(dqProbs)
        , mUseInt8ScaleMax(useInt8ScaleMax ? 1 : 0)
        , mUseExplicitInt8(useExplicitInt8 ? 1 : 0)
        , mQkvScale(qkvScale)
        , mCtxScale(ctxScale)
    {
        mSM = getSmVersion();
        prepareFusedKernels(DataType::kINT8);
    }

protected:
    std::unique_ptr<BertPluginBase> doClone() override
    {
        return std::make_unique<QkvToContextInterleavedPlugin>(mLayerName, mHiddenSize, mNumHeads, mDqProbs,
            mUseInt8ScaleMax != 0, mUseExplicitInt8 != 0, mQkvScale, mCtxScale);
    }

    void doOutputTypes(DataType* outputTypes, DataType const*) const override
    {
        outputTypes[0] = DataType::kINT8;
    }

    void doOutputShapes(DimsExprs const* inputs, DimsExprs* outputs, IExprBuilder& eb) override
    {
        // [1, 3*N*H, total, 1] -> [1, N*H, total, 1]; with kCHW32 the bytes are [3][N][H/32][total][32]
        outputs[0] = inputs[kIIDX];
        outputs[0].d[1] = eb.operation(DimensionOperation::kFLOOR_DIV, *inputs[kIIDX].d[1], *eb.constant(3));
    }

    bool doSupportsFormat(int32_t pos, DynamicPluginTensorDesc const* inOut) override
    {
        if (pos == 0 || pos == mNbInputs)
        {
            return inOut[pos].desc.type == DataType::kINT8 && inOut[pos].desc.format == TensorFormat::kCHW32;
        }
        if (pos == 1) // cu_seqlens, B + 1 entries
        {
            return inOut[pos].desc.type == DataType::kINT32 && inOut[pos].desc.format == TensorFormat::kLINEAR;
        }
        if (pos == 2) // dummy input whose extent is the maximum sequence length
        {
            return inOut[pos].desc.dims.nbDims == 1;
        }
        return false;
    }

    int32_t doEnqueue(PluginTensorDesc const* inputDesc, PluginTensorDesc const* outputDesc, void const* const* inputs,
        void* const* outputs, void*, hipStream_t stream) override
    {
        int32_t const total = static_cast<int32_t>(inputDesc[0].dims.d[2]);
        int32_t const B = static_cast<int32_t>(inputDesc[1].dims.d[0]) - 1;
        int32_t const maxS = static_cast<int32_t>(inputDesc[2].dims.d[0]);
        // The reference has interleaved kernels for 128, 192, 256 and 384 keys only and silently
        // uses the 384 one beyond; here up to 512 keys are served and longer input is an error.
        int32_t S = maxS <= 128 ? 128 : maxS <= 192 ? 192 : maxS <= 256 ? 256 : maxS <= 384 ? 384 : maxS;
        trtamd_fmha_params p{};
        p.b = B;
        p.s = S;
        p.h = mNumHeads;
        p.d = mHeadSize;
        p.interleaved = 1;
        p.o_ptr = outputs[0];
        p.qkv_ptr = inputs[0];
        p.cu_seqlens = static_cast<int32_t const*>(inputs[1]);
        float const scaleQkv = mUseExplicitInt8 ? mQkvScale : inputDesc[0].scale;
        float const scaleCtx = mUseExplicitInt8 ? mCtxScale : outputDesc[0].scale;
        // 0.125 = 1/sqrt(64) is hard-wired in the reference (qkvToContextInt8InterleavedPlugin.cpp:272)
        fillInt8Scales(p, scaleQkv, scaleCtx, 0.125F, mDqProbs);
        p.qkv_stride_in_bytes = total;
        p.o_stride_in_bytes = total;
        p.use_int8_scale_max = mUseInt8ScaleMax;
        checkKernelStatus(trtamd_fused_mha_run(stream, static_cast<int32_t>(DataType::kINT8), &p), "fused attention");
        return 0;
    }

    void doSerialize(FieldList& f) override
    {
        f.add("hidden_size", &mHiddenSize, PluginFieldType::kINT32, 1);
        f.add("num_heads", &mNumHeads, PluginFieldType::kINT32, 1);
        f.add("use_int8_scale_max", &mUseInt8ScaleMax, PluginFieldType::kINT32, 1);
        f.add("use_explicit_int8", &mUseExplicitInt8, PluginFieldType::kINT32, 1);
        f.add("input_qkv_scale", &mQkvScale, PluginFieldType::kFLOAT32, 1);
        f.add("output_ctx_scale", &mCtxScale, PluginFieldType::kFLOAT32, 1);
        if (mDqProbs >= 0)
        {
            f.add("dq_probs", &mDqProbs, PluginFieldType::kFLOAT32, 1);
        }
    }

private:
    int32_t mSM{0};
    int32_t mHeadSize;
    int32_t mHiddenSize;
    int32_t mNumHeads;
    float mDqProbs;
    int32_t mUseInt8ScaleMax;
    int32_t mUseExplicitInt8;
    float mQkvScale;
    float mCtxScale;
};

class QkvToContextInterleavedCreator final : public BertCreatorBase
{
public:
    QkvToContextInterleavedCreator()
        : BertCreatorBase(kNAME, "6",
            {PluginField("hidden_size", nullptr, PluginFieldType::kINT32, 1),
                PluginField("num_heads", nullptr, PluginFieldType::kINT32, 1),
                PluginField("dq_probs", nullptr, PluginFieldType::kFLOAT32, 1),
                PluginField("use_int8_scale_max", nullptr, PluginFieldType::kINT32, 1),
                PluginField("use_explicit_int8", nullptr, PluginFieldType::kINT32, 1),
                PluginField("input_qkv_scale", nullptr, PluginFieldType::kFLOAT32, 1),
                PluginField("output_ctx_scale", nullptr, PluginFieldType::kFLOAT32, 1)})
    {
    }

protected:
    std::unique_ptr<BertPluginBase> doCreate(char const* name, PluginFieldCollection const* fc,
        TensorRTPhase phase) override
    {
        if (phase == TensorRTPhase::kBUILD)
        {
            validateRequiredFields({"hidden_size", "num_heads"}, fc);
        }
        else
        {
            validateRequiredFields({"hidden_size", "num_heads", "use_int8_scale_max", "use_explicit_int8",
                                       "input_qkv_scale", "output_ctx_scale"},
                fc);
        }
        int32_t hiddenSize = 0;
        int32_t numHeads = -1;
        float dqProbs = 1.F / 127.F;
        int32_t useInt8ScaleMax = 1;
        int32_t useExplicitInt8 = 0;
        float qkvScale = 1.F;
        float ctxScale = 1.F;
        if (readScalar(fc, "hidden_size", hiddenSize))
        {
            TRTAMD_VALIDATE_MSG(hiddenSize > 0, "QKV: Invalid hiddenSize " + std::to_string(hiddenSize));
        }
        if (readScalar(fc, "num_heads", numHeads))
        {
            TRTAMD_VALIDATE_MSG(numHeads > 0, "QKV: Invalid numHeads " + std::to_string(numHeads));
        }
        if (readScalar(fc, "dq_probs", dqProbs))
        {
            TRTAMD_VALIDATE_MSG(dqProbs > 0.0F, "QKV: Invalid dqProbs " + std::to_string(dqProbs));
        }
        if (readScalar(fc, "use_int8_scale_max", useInt8ScaleMax))
        {
            TRTAMD_VALIDATE_MSG(useInt8ScaleMax == 0 || useInt8ScaleMax == 1,
                "QKV: Invalid useInt8ScaleMax " + std::to_string(useInt8ScaleMax));
        }
        if (readScalar(fc, "use_explicit_int8", useExplicitInt8))
        {
            TRTAMD_VALIDATE_MSG(useExplicitInt8 == 0 || useExplicitInt8 == 1,
                "QKV: Invalid useExplicitInt8 " + std::to_string(useExplicitInt8));
        }
        if (readScalar(fc, "input_qkv_scale", qkvScale))
        {
            TRTAMD_VALIDATE_MSG(qkvScale > 0, "QKV: Invalid input_qkv_scale" + std::to_string(qkvScale));
        }
        if (readScalar(fc, "output_ctx_scale", ctxScale))
        {
            TRTAMD_VALIDATE_MSG(ctxScale > 0, "QKV: Invalid output_ctx_scale " + std::to_string(ctxScale));
        }
        return std::make_unique<QkvToContextInterleavedPlugin>(name, hiddenSize, numHeads, dqProbs,
            useInt8ScaleMax != 0, useExplicitInt8 != 0, qkvScale, ctxScale);
    }
};

REGISTER_TENSORRT_PLUGIN(QkvToContextCreator);
REGISTER_TENSORRT_PLUGIN(QkvToContextVarSeqlenCreator);
REGISTER_TENSORRT_PLUGIN(QkvToContextInterleavedCreator);

} // namespace
} // namespace plugin
} // namespace trtamd
