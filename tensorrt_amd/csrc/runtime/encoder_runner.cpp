// Native runner of a built INT8 BERT encoder (include/trtamd_encoder_runtime.h): what a deserialised engine
// holds (runtime-phase plugin objects from the registry, device weights, activation scales) and the
// stream-ordered sequence of plugin enqueues and linear layers that executes it.  enqueue() only launches, the
// first call included: every device allocation, copy and kernel attribute happens in set_embedding / set_layer
// (which run each plugin's first shape change), the activations live in the caller's workspace.
// Execution contexts (reserve_contexts) are further sets of the plugin objects, cloned, each with a stream and two
// events; enqueue_concurrent runs one batch per context at the same time, forked from and joined to the caller's
// stream, and launches the batches' steps in turn so that every stream is fed from the start.
#include "plugin_common.h"
#include "trtamd_encoder_runtime.h"

#include "../host_utils.hpp"

#include <memory>
#include <string>
#include <vector>

namespace trtamd
{
namespace runtime
{
namespace
{

using namespace trtamd::plugin;

constexpr char const* kEMB = "CustomEmbLayerNormPluginDynamic";
constexpr char const* kSKIP = "CustomSkipLayerNormPluginDynamic";
constexpr char const* kQKV = "CustomQKVToContextPluginDynamic";

struct PluginDeleter
{
    void operator()(IPluginV3* p) const
    {
        delete p;
    }
};
using PluginPtr = std::unique_ptr<IPluginV3, PluginDeleter>;

// Build-phase plugin -> serialised fields -> runtime-phase plugin, the round trip an engine file makes.
PluginPtr makeRuntimePlugin(char const* name, char const* version, std::string const& layer,
    std::vector<PluginField> const& fields)
{
    auto* creator = static_cast<IPluginCreatorV3One*>(getPluginRegistry()->getCreator(name, version, ""));
    TRTAMD_VALIDATE_MSG(creator != nullptr, std::string(name) + " version " + version + " is not registered");
    PluginFieldCollection fc{static_cast<int32_t>(fields.size()), fields.data()};
    PluginPtr built(creator->createPlugin(layer.c_str(), &fc, TensorRTPhase::kBUILD));
    TRTAMD_VALIDATE_MSG(built != nullptr, layer + ": createPlugin failed");
    auto* rt = static_cast<IPluginV3OneRuntime*>(built->getCapabilityInterface(PluginCapabilityType::kRUNTIME));
    PluginFieldCollection const* ser = rt->getFieldsToSerialize();
    TRTAMD_VALIDATE_MSG(ser != nullptr, layer + ": getFieldsToSerialize failed");
    PluginPtr runtime(creator->createPlugin(layer.c_str(), ser, TensorRTPhase::kRUNTIME));
    TRTAMD_VALIDATE_MSG(runtime != nullptr, layer + ": runtime createPlugin failed");
    return runtime;
}

IPluginV3OneRuntime* runtimeOf(PluginPtr const& p)
{
    return static_cast<IPluginV3OneRuntime*>(p->getCapabilityInterface(PluginCapabilityType::kRUNTIME));
}

PluginTensorDesc desc(std::initializer_list<int64_t> dims, DataType type, TensorFormat format, float scale)
{
    PluginTensorDesc d{};
    d.dims.nbDims = static_cast<int32_t>(dims.size());
    int32_t i = 0;
    for (int64_t v : dims)
    {
        d.dims.d[i++] = v;
    }
    d.type = type;
    d.format = format;
    d.scale = scale;
    return d;
}

// One INT8 fully-connected layer resident on the GPU: weights in the interleaved layout, folded scales.
struct LinearLayer
{
    DeviceBuffer w, alpha, beta;
    int32_t N{0}, K{0};

    void load(trtamd_encoder_linear const& src, int32_t n, int32_t k)
    {
        TRTAMD_VALIDATE(src.w != nullptr && src.alpha != nullptr && src.beta != nullptr);
        N = n;
        K = k;
        DeviceBuffer linear;
        linear.upload(src.w, static_cast<size_t>(n) * k);
        w.upload(src.w, static_cast<size_t>(n) * k); // allocation of the right size; overwritten below
        checkKernelStatus(trtamd_int8_linear_to_interleaved(nullptr, n, k, linear.as<int8_t>(),
                              static_cast<int8_t*>(w.get())),
            "weight reformat");
        TRTAMD_VALIDATE(hipStreamSynchronize(nullptr) == hipSuccess); // `linear` is freed on return
        alpha.upload(src.alpha, sizeof(float) * n);
        beta.upload(src.beta, sizeof(float) * n);
    }

    int run(hipStream_t stream, int8_t const* a, int8_t* out, int32_t tokens, int32_t epilogue, float outScale) const
    {
        trtamd_int8_linear_params p{};
        p.a = a;
        p.w = w.as<int8_t>();
        p.alpha = alpha.as<float>();
        p.beta = beta.as<float>();
        p.out = out;
        p.T = tokens;
        p.K = K;
        p.N = N;
        p.a_interleaved = p.w_interleaved = p.out_interleaved = 1;
        p.epilogue = epilogue;
        p.out_scale = outScale;
        return trtamd_int8_linear(stream, &p);
    }
};

// The plugin objects of one layer.  They keep per-shape state between onShapeChange and enqueue, so every execution
// context has a set of its own (clones of the first one, as TensorRT clones an engine's plugins for each
// IExecutionContext it creates).
struct LayerPlugins
{
    PluginPtr attention, ln1, ln2;
};

struct Layer
{
    LinearLayer qkv, proj, ffn1, ffn2;
    float ffn1OutScale{1.f};
    float sX{0}, sQkv{0}, sCtx{0}, sAo{0}, sH{0}, sF{0}, sOut{0};
    bool set{false};
};

size_t align256(size_t n)
{
    return (n + 255) & ~size_t(255);
}

class Encoder
{
public:
    explicit Encoder(trtamd_encoder_config const& c)
        : mCfg(c)
        , mLayers(static_cast<size_t>(c.layers))
    {
        TRTAMD_VALIDATE_MSG(c.hidden > 0 && c.heads > 0 && c.hidden == c.heads * 64,
            "the INT8 interleaved attention plugin serves heads of 64 channels");
        TRTAMD_VALIDATE(c.hidden % 64 == 0 && c.ffn % 64 == 0 && c.ffn > 0 && c.layers >= 0);
        TRTAMD_VALIDATE(c.vocab > 0 && c.max_pos > 0 && c.type_vocab > 0 && c.max_seqlen > 0 && c.max_seqlen <= 512);
        mContexts.resize(1);
        mContexts[0].layers.resize(static_cast<size_t>(c.layers));
    }

    Encoder(Encoder const&) = delete;
    Encoder& operator=(Encoder const&) = delete;

    void setEmbedding(trtamd_encoder_embedding const& e)
    {
        TRTAMD_VALIDATE(e.beta && e.gamma && e.word && e.tok && e.pos && e.scale > 0.f);
        int32_t const E = mCfg.hidden;
        int32_t const fp16 = 1;
        std::vector<PluginField> f{
            {"bert_embeddings_layernorm_beta", e.beta, PluginFieldType::kFLOAT32, E},
            {"bert_embeddings_layernorm_gamma", e.gamma, PluginFieldType::kFLOAT32, E},
            {"bert_embeddings_word_embeddings", e.word, PluginFieldType::kFLOAT32, mCfg.vocab * E},
            {"bert_embeddings_token_type_embeddings", e.tok, PluginFieldType::kFLOAT32, mCfg.type_vocab * E},
            {"bert_embeddings_position_embeddings", e.pos, PluginFieldType::kFLOAT32, mCfg.max_pos * E},
            {"output_fp16", &fp16, PluginFieldType::kINT32, 1}};
        TRTAMD_VALIDATE_MSG(mContexts.size() == 1, "set_embedding after reserve_contexts");
        mContexts[0].embedding = makeRuntimePlugin(kEMB, "4", "embeddings", f);
        mEmbScale = e.scale;
    }

    void setLayer(int32_t index, trtamd_encoder_layer const& l)
    {
        TRTAMD_VALIDATE_MSG(index >= 0 && index < mCfg.layers, "layer index out of range");
        TRTAMD_VALIDATE(l.ln1_gamma && l.ln1_beta && l.ln2_gamma && l.ln2_beta);
        TRTAMD_VALIDATE(l.s_x > 0 && l.s_qkv > 0 && l.s_ctx > 0 && l.s_ao > 0 && l.s_h > 0 && l.s_f > 0 && l.s_out > 0);
        TRTAMD_VALIDATE_MSG(mContexts.size() == 1, "set_layer after reserve_contexts");
        int32_t const E = mCfg.hidden, F = mCfg.ffn;
        Layer& L = mLayers[static_cast<size_t>(index)];
        LayerPlugins& P = mContexts[0].layers[static_cast<size_t>(index)];
        L.qkv.load(l.qkv, 3 * E, E);
        L.proj.load(l.proj, E, E);
        L.ffn1.load(l.ffn1, F, E);
        L.ffn2.load(l.ffn2, E, F);
        L.ffn1OutScale = l.ffn1_out_scale;
        std::string const tag = "l" + std::to_string(index);
        float const dqProbs = 1.f / 127.f;
        std::vector<PluginField> qf{{"hidden_size", &mCfg.hidden, PluginFieldType::kINT32, 1},
            {"num_heads", &mCfg.heads, PluginFieldType::kINT32, 1}, {"dq_probs", &dqProbs, PluginFieldType::kFLOAT32, 1}};
        P.attention = makeRuntimePlugin(kQKV, "6", tag + "_attention", qf);
        auto ln = [&](char const* which, trtamd_half_t const* gamma, trtamd_half_t const* beta) {
            std::vector<PluginField> f{{"beta", beta, PluginFieldType::kFLOAT16, E}, {"gamma", gamma, PluginFieldType::kFLOAT16, E}};
            return makeRuntimePlugin(kSKIP, "7", tag + which, f);
        };
        P.ln1 = ln("_ln1", l.ln1_gamma, l.ln1_beta);
        P.ln2 = ln("_ln2", l.ln2_gamma, l.ln2_beta);
        firstShapeChange(P, tag);
        L.sX = l.s_x;
        L.sQkv = l.s_qkv;
        L.sCtx = l.s_ctx;
        L.sAo = l.s_ao;
        L.sH = l.s_h;
        L.sF = l.s_f;
        L.sOut = l.s_out;
        L.set = true;
    }

    // One shape change with representative descriptors, so that whatever a plugin sets up on its first shape change
    // (device copies of parameters, kernel attributes) is done before the first enqueue, which a caller may be
    // recording into a graph.
    void firstShapeChange(LayerPlugins const& P, std::string const& tag) const
    {
        int64_t const T = mCfg.max_seqlen, E = mCfg.hidden;
        auto const il = TensorFormat::kCHW32;
        auto const lin = TensorFormat::kLINEAR;
        PluginTensorDesc const act = desc({1, E, T, 1}, DataType::kINT8, il, 1.f);
        PluginTensorDesc const lnIn[2] = {act, act};
        for (PluginPtr const* p : {&P.ln1, &P.ln2})
        {
            TRTAMD_VALIDATE_MSG(runtimeOf(*p)->onShapeChange(lnIn, 2, &act, 1) == 0, tag + ": SkipLayerNorm set-up failed");
        }
        PluginTensorDesc const qIn[3] = {desc({1, 3 * E, T, 1}, DataType::kINT8, il, 1.f),
            desc({2}, DataType::kINT32, lin, 1.f), desc({T}, DataType::kINT32, lin, 1.f)};
        TRTAMD_VALIDATE_MSG(runtimeOf(P.attention)->onShapeChange(qIn, 3, &act, 1) == 0, tag + ": attention set-up failed");
    }

    // Execution contexts beyond the first: clones of every plugin object (IPluginV3::clone, what TensorRT does for
    // each IExecutionContext of an engine), and for each of them a stream and two events of the runner's own, so
    // that enqueueConcurrent has nothing left to create.  Weights and scales are shared.
    void reserveContexts(int32_t count)
    {
        TRTAMD_VALIDATE_MSG(count >= 1 && count <= kMaxContexts, "between 1 and 8 execution contexts");
        requireComplete();
        while (static_cast<int32_t>(mContexts.size()) < count)
        {
            Context c;
            Context const& first = mContexts[0];
            auto cloneOf = [](PluginPtr const& p, char const* what) {
                PluginPtr q(p->clone());
                TRTAMD_VALIDATE_MSG(q != nullptr, std::string(what) + ": clone failed");
                return q;
            };
            c.embedding = cloneOf(first.embedding, "EmbLayerNorm");
            c.layers.resize(first.layers.size());
            for (size_t i = 0; i < first.layers.size(); ++i)
            {
                c.layers[i].attention = cloneOf(first.layers[i].attention, "QKV-to-context");
                c.layers[i].ln1 = cloneOf(first.layers[i].ln1, "SkipLayerNorm 1");
                c.layers[i].ln2 = cloneOf(first.layers[i].ln2, "SkipLayerNorm 2");
                firstShapeChange(c.layers[i], "context " + std::to_string(mContexts.size()) + " l" + std::to_string(i));
            }
            // default priority, no implicit synchronisation with the null stream
            TRTAMD_VALIDATE_MSG(hipStreamCreateWithFlags(&c.side.stream, hipStreamNonBlocking) == hipSuccess,
                "cannot create a stream for an execution context");
            TRTAMD_VALIDATE(hipEventCreateWithFlags(&c.side.fork, hipEventDisableTiming) == hipSuccess);
            TRTAMD_VALIDATE(hipEventCreateWithFlags(&c.side.join, hipEventDisableTiming) == hipSuccess);
            mContexts.push_back(std::move(c));
        }
    }

    int32_t contexts() const
    {
        return static_cast<int32_t>(mContexts.size());
    }

    // emb fp16 | x | qkv | ctx | ao | h | m | f | dummy | emb's second output
    size_t workspaceSize(int32_t tokens) const
    {
        size_t const T = static_cast<size_t>(tokens > 0 ? tokens : 0);
        size_t const E = static_cast<size_t>(mCfg.hidden), F = static_cast<size_t>(mCfg.ffn);
        return align256(T * E * 2) + 5 * align256(T * E) + align256(3 * T * E) + align256(T * F)
            + align256(sizeof(int32_t) * static_cast<size_t>(mCfg.max_seqlen)) + 256;
    }

    int enqueue(int32_t const* ids, int32_t const* segs, int32_t const* cu, int32_t batch, int32_t tokens,
        void* workspace, trtamd_half_t* out, hipStream_t stream)
    {
        requireComplete();
        trtamd_encoder_batch const whole{ids, segs, cu, batch, tokens, workspace, out};
        Pass pass(*this, mContexts[0], whole, stream);
        pass.embed();
        for (size_t li = 0; li < mLayers.size(); ++li)
        {
            pass.layer(li);
        }
        pass.finish();
        return TRTAMD_STATUS_SUCCESS;
    }

    // Several independent batches at once: part 0 on the caller's stream, part i on the stream of context i, which
    // starts behind everything the caller's stream holds so far (fork event) and which the caller's stream waits for
    // before anything enqueued after this call (join event).  To the caller the whole call is work on `stream`; it
    // only launches and records, so it can be captured into a graph like the single enqueue.
    int enqueueConcurrent(trtamd_encoder_batch const* parts, int32_t count, hipStream_t stream)
    {
        requireComplete();
        TRTAMD_VALIDATE_MSG(parts != nullptr && count >= 1, "at least one part is required");
        TRTAMD_VALIDATE_MSG(count <= contexts(),
            "more parts than reserved execution contexts (trtamd_encoder_reserve_contexts)");
        std::vector<Pass> passes;
        passes.reserve(static_cast<size_t>(count));
        for (int32_t i = 0; i < count; ++i)
        {
            Context& c = mContexts[static_cast<size_t>(i)];
            passes.emplace_back(*this, c, parts[i], i == 0 ? stream : c.side.stream);
        }
        // arguments are checked (above) before anything is recorded, so that a refused call leaves no stream forked;
        // if forking fails half way, the streams forked so far are joined again before the error leaves
        int32_t forked = 1;
        auto join = [&] {
            bool ok = true;
            for (int32_t i = 1; i < forked; ++i)
            {
                Side const& sd = mContexts[static_cast<size_t>(i)].side;
                ok = hipEventRecord(sd.join, sd.stream) == hipSuccess && ok;
                ok = hipStreamWaitEvent(stream, sd.join, 0) == hipSuccess && ok;
            }
            return ok;
        };
        try
        {
            for (int32_t i = 1; i < count; ++i)
            {
                Side const& sd = mContexts[static_cast<size_t>(i)].side;
                TRTAMD_VALIDATE(hipEventRecord(sd.fork, stream) == hipSuccess);
                TRTAMD_VALIDATE(hipStreamWaitEvent(sd.stream, sd.fork, 0) == hipSuccess);
                forked = i + 1;
            }
            for (Pass& p : passes)
            {
                p.embed();
            }
            for (size_t li = 0; li < mLayers.size(); ++li)
            {
                for (Pass& p : passes)
                {
                    p.layer(li);
                }
            }
            for (Pass& p : passes)
            {
                p.finish();
            }
        }
        catch (...)
        {
            (void) join(); // a forked stream is joined whatever happened in between
            throw;
        }
        TRTAMD_VALIDATE_MSG(join(), "cannot join the execution contexts' streams");
        return TRTAMD_STATUS_SUCCESS;
    }

private:
    static constexpr int32_t kMaxContexts = 8;

    // The stream and the two events of a context beyond the first; owns them.
    struct Side
    {
        hipStream_t stream{nullptr};
        hipEvent_t fork{nullptr}, join{nullptr};

        Side() = default;
        Side(Side const&) = delete;
        Side& operator=(Side const&) = delete;
        Side(Side&& o) noexcept : stream(o.stream), fork(o.fork), join(o.join)
        {
            o.stream = nullptr;
            o.fork = o.join = nullptr;
        }
        Side& operator=(Side&& o) noexcept
        {
            if (this != &o)
            {
                release();
                stream = o.stream, fork = o.fork, join = o.join;
                o.stream = nullptr;
                o.fork = o.join = nullptr;
            }
            return *this;
        }
        ~Side()
        {
            release();
        }
        void release() noexcept
        {
            if (stream)
            {
                (void) hipStreamSynchronize(stream);
                (void) hipStreamDestroy(stream);
            }
            if (fork)
            {
                (void) hipEventDestroy(fork);
            }
            if (join)
            {
                (void) hipEventDestroy(join);
            }
            stream = nullptr;
            fork = join = nullptr;
        }
    };

    struct Context
    {
        PluginPtr embedding;
        std::vector<LayerPlugins> layers;
        Side side;
    };

    void requireComplete() const
    {
        TRTAMD_VALIDATE_MSG(mContexts[0].embedding != nullptr, "set_embedding has not been called");
        for (Layer const& L : mLayers)
        {
            TRTAMD_VALIDATE_MSG(L.set, "set_layer has not been called for every layer");
        }
    }

    // One batch on its way through the network: the buffers carved out of its workspace and the three kinds of step
    // (embedding, one layer, output).  A single enqueue walks the steps in order; the concurrent one takes the steps of
    // its parts in turn, layer by layer, so that every stream has work from the first few launches on instead of
    // part 1 waiting on the host until all of part 0 has been launched.
    struct Pass
    {
        Encoder const& enc;
        Context& context;
        hipStream_t stream;
        int32_t const* ids;
        int32_t const* segs;
        int32_t const* cu;
        int64_t T, B;
        trtamd_half_t* emb;
        int8_t *x, *qkv, *ctx, *ao, *h, *m, *f;
        uint8_t *dummy, *emb2;
        trtamd_half_t* out;
        float lastScale;

        Pass(Encoder const& e, Context& c, trtamd_encoder_batch const& b, hipStream_t s)
            : enc(e), context(c), stream(s), ids(b.ids), segs(b.segment_ids), cu(b.cu_seqlens), T(b.tokens), B(b.batch),
              out(b.out), lastScale(e.mEmbScale)
        {
            TRTAMD_VALIDATE(ids && segs && cu && b.workspace && out && b.batch > 0 && b.tokens > 0);
            TRTAMD_VALIDATE_MSG((reinterpret_cast<uintptr_t>(b.workspace) & 255u) == 0, "workspace must be 256-byte aligned");
            int64_t const E = enc.mCfg.hidden, F = enc.mCfg.ffn;
            auto* base = static_cast<uint8_t*>(b.workspace);
            auto carve = [&](size_t bytes) {
                uint8_t* p = base;
                base += align256(bytes);
                return p;
            };
            emb = reinterpret_cast<trtamd_half_t*>(carve(T * E * 2));
            x = reinterpret_cast<int8_t*>(carve(T * E));
            qkv = reinterpret_cast<int8_t*>(carve(3 * T * E));
            ctx = reinterpret_cast<int8_t*>(carve(T * E));
            ao = reinterpret_cast<int8_t*>(carve(T * E));
            h = reinterpret_cast<int8_t*>(carve(T * E));
            m = reinterpret_cast<int8_t*>(carve(T * F));
            f = reinterpret_cast<int8_t*>(carve(T * E));
            dummy = carve(sizeof(int32_t) * static_cast<size_t>(enc.mCfg.max_seqlen)); // only its extent is read
            emb2 = carve(256);
        }

        void run(PluginPtr const& plugin, std::vector<PluginTensorDesc> const& in,
            std::vector<PluginTensorDesc> const& outDesc, std::vector<void const*> const& inputs,
            std::vector<void*> const& outputs, char const* what) const
        {
            IPluginV3OneRuntime* rt = runtimeOf(plugin);
            int32_t st = rt->onShapeChange(in.data(), static_cast<int32_t>(in.size()), outDesc.data(),
                static_cast<int32_t>(outDesc.size()));
            if (st == 0)
            {
                st = rt->enqueue(in.data(), outDesc.data(), inputs.data(), outputs.data(), nullptr, stream);
            }
            TRTAMD_VALIDATE_MSG(st == 0, std::string(what) + " failed with status " + std::to_string(st));
        }

        void embed()
        {
            auto const lin = TensorFormat::kLINEAR;
            int64_t const E = enc.mCfg.hidden;
            run(context.embedding,
                {desc({T}, DataType::kINT32, lin, 1.f), desc({T}, DataType::kINT32, lin, 1.f),
                    desc({B + 1}, DataType::kINT32, lin, 1.f), desc({enc.mCfg.max_seqlen}, DataType::kINT32, lin, 1.f)},
                {desc({T, E, 1, 1}, DataType::kHALF, lin, 1.f), desc({}, DataType::kINT32, lin, 1.f)},
                {ids, segs, cu, dummy}, {emb, emb2}, "EmbLayerNorm");
            checkKernelStatus(trtamd_quantize_fp16_to_interleaved(stream, static_cast<int32_t>(T), enc.mCfg.hidden, emb,
                                  enc.mEmbScale, x),
                "quantise");
        }

        void layer(size_t li)
        {
            auto const lin = TensorFormat::kLINEAR;
            auto const il = TensorFormat::kCHW32;
            int64_t const E = enc.mCfg.hidden;
            int32_t const tokens = static_cast<int32_t>(T);
            Layer const& L = enc.mLayers[li];
            LayerPlugins const& P = context.layers[li];
            checkKernelStatus(L.qkv.run(stream, x, qkv, tokens, TRTAMD_LINEAR_AFFINE, 1.f), "QKV projection");
            run(P.attention,
                {desc({1, 3 * E, T, 1}, DataType::kINT8, il, L.sQkv), desc({B + 1}, DataType::kINT32, lin, 1.f),
                    desc({enc.mCfg.max_seqlen}, DataType::kINT32, lin, 1.f)},
                {desc({1, E, T, 1}, DataType::kINT8, il, L.sCtx)}, {qkv, cu, dummy}, {ctx}, "QKV-to-context");
            checkKernelStatus(L.proj.run(stream, ctx, ao, tokens, TRTAMD_LINEAR_AFFINE, 1.f), "output projection");
            run(P.ln1, {desc({1, E, T, 1}, DataType::kINT8, il, L.sAo), desc({1, E, T, 1}, DataType::kINT8, il, L.sX)},
                {desc({1, E, T, 1}, DataType::kINT8, il, L.sH)}, {ao, x}, {h}, "SkipLayerNorm 1");
            checkKernelStatus(L.ffn1.run(stream, h, m, tokens, TRTAMD_LINEAR_GELU, L.ffn1OutScale), "feed-forward 1");
            checkKernelStatus(L.ffn2.run(stream, m, f, tokens, TRTAMD_LINEAR_AFFINE, 1.f), "feed-forward 2");
            run(P.ln2, {desc({1, E, T, 1}, DataType::kINT8, il, L.sF), desc({1, E, T, 1}, DataType::kINT8, il, L.sH)},
                {desc({1, E, T, 1}, DataType::kINT8, il, L.sOut)}, {f, h}, {x}, "SkipLayerNorm 2");
            lastScale = L.sOut;
        }

        void finish()
        {
            checkKernelStatus(trtamd_dequantize_interleaved_to_fp16(stream, static_cast<int32_t>(T), enc.mCfg.hidden, x,
                                  lastScale, out),
                "dequantise");
        }
    };

    trtamd_encoder_config mCfg;
    float mEmbScale{0.f};
    std::vector<Layer> mLayers;
    std::vector<Context> mContexts; // [0]: the plugin objects set_embedding / set_layer create
};

template <typename Fn>
int guarded(char const* what, Fn&& fn)
{
    try
    {
        return fn();
    }
    catch (std::exception const& e)
    {
        return set_error(TRTAMD_STATUS_FAILURE, "%s: %s", what, e.what());
    }
}

} // namespace
} // namespace runtime
} // namespace trtamd

using trtamd::runtime::Encoder;
using trtamd::runtime::guarded;

extern "C" trtamd_encoder_t trtamd_encoder_create(trtamd_encoder_config const* config)
{
    Encoder* enc = nullptr;
    guarded("encoder_create", [&] {
        TRTAMD_VALIDATE(config != nullptr);
        enc = new Encoder(*config);
        return 0;
    });
    return enc;
}

extern "C" void trtamd_encoder_destroy(trtamd_encoder_t encoder)
{
    delete static_cast<Encoder*>(encoder);
}

extern "C" int trtamd_encoder_set_embedding(trtamd_encoder_t encoder, trtamd_encoder_embedding const* embedding)
{
    return guarded("encoder_set_embedding", [&] {
        TRTAMD_VALIDATE(encoder != nullptr && embedding != nullptr);
        static_cast<Encoder*>(encoder)->setEmbedding(*embedding);
        return 0;
    });
}

extern "C" int trtamd_encoder_set_layer(trtamd_encoder_t encoder, int32_t index, trtamd_encoder_layer const* layer)
{
    return guarded("encoder_set_layer", [&] {
        TRTAMD_VALIDATE(encoder != nullptr && layer != nullptr);
        static_cast<Encoder*>(encoder)->setLayer(index, *layer);
        return 0;
    });
}

extern "C" size_t trtamd_encoder_workspace_size(trtamd_encoder_t encoder, int32_t max_tokens)
{
    return encoder ? static_cast<Encoder*>(encoder)->workspaceSize(max_tokens) : 0;
}

extern "C" int trtamd_encoder_enqueue(trtamd_encoder_t encoder, int32_t const* ids, int32_t const* segment_ids,
    int32_t const* cu_seqlens, int32_t batch, int32_t tokens, void* workspace, trtamd_half_t* out,
    trtamd_stream_t stream)
{
    return guarded("encoder_enqueue", [&] {
        TRTAMD_VALIDATE(encoder != nullptr);
        return static_cast<Encoder*>(encoder)->enqueue(ids, segment_ids, cu_seqlens, batch, tokens, workspace, out,
            trtamd::as_stream(stream));
    });
}

extern "C" int trtamd_encoder_reserve_contexts(trtamd_encoder_t encoder, int32_t count)
{
    return guarded("encoder_reserve_contexts", [&] {
        TRTAMD_VALIDATE(encoder != nullptr);
        static_cast<Encoder*>(encoder)->reserveContexts(count);
        return 0;
    });
}

extern "C" int trtamd_encoder_enqueue_concurrent(trtamd_encoder_t encoder, trtamd_encoder_batch const* parts,
    int32_t count, trtamd_stream_t stream)
{
    return guarded("encoder_enqueue_concurrent", [&] {
        TRTAMD_VALIDATE(encoder != nullptr);
        return static_cast<Encoder*>(encoder)->enqueueConcurrent(parts, count, trtamd::as_stream(stream));
    });
}
