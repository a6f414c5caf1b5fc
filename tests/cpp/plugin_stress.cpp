// Host-side robustness of the plugin library, for a build of its host sources with AddressSanitizer and
// UndefinedBehaviorSanitizer (tests/test_host_sanitizers.py; it runs as well against the plain library):
//   threads: eight threads create, clone, serialise, deserialise and destroy plugins of every family at the same time
//            (the reference guards its creators with a mutex, plugin/skipLayerNormPlugin/skipLayerNormPlugin.cpp:441-453);
//   fuzz:    every legacy creator's deserializePlugin on truncated, bit-flipped, length-corrupted and random streams:
//            each call must return a plugin or nullptr, never crash or read outside the buffer (the buffers are exact-size
//            heap blocks, so the sanitizer sees any overrun).
// Prints "ok" and returns 0 when every check holds.  Nothing here launches a kernel.
#include "trtamd_nvinfer_api.h"

#include <atomic>
#include <cstdio>
#include <cstring>
#include <memory>
#include <random>
#include <string>
#include <thread>
#include <vector>

using namespace nvinfer1;

namespace
{
class QuietLogger final : public ILogger
{
public:
    void log(Severity, AsciiChar const*) noexcept override {}
};

struct Fields
{
    // owns the values the PluginFields point at
    std::vector<std::vector<float>> floats;
    std::vector<int32_t> ints;
    std::vector<PluginField> fields;
    PluginFieldCollection fc{};

    void addFloats(char const* name, size_t n, float v)
    {
        floats.emplace_back(n, v);
        pending.push_back({name, floats.size() - 1, true, n});
    }
    void addInt(char const* name, int32_t v)
    {
        ints.push_back(v);
        pending.push_back({name, ints.size() - 1, false, 1});
    }
    void addFloat(char const* name, float v)
    {
        addFloats(name, 1, v);
    }
    PluginFieldCollection const* finish()
    {
        ints.shrink_to_fit();
        fields.clear();
        for (auto const& p : pending)
        {
            if (p.isFloat)
            {
                fields.push_back({p.name, floats[p.index].data(), PluginFieldType::kFLOAT32, static_cast<int32_t>(p.n)});
            }
            else
            {
                fields.push_back({p.name, &ints[p.index], PluginFieldType::kINT32, 1});
            }
        }
        fc = {static_cast<int32_t>(fields.size()), fields.data()};
        return &fc;
    }

private:
    struct Pending
    {
        char const* name;
        size_t index;
        bool isFloat;
        size_t n;
    };
    std::vector<Pending> pending;
};

char const* const kSkip = "CustomSkipLayerNormPluginDynamic";
char const* const kEmb = "CustomEmbLayerNormPluginDynamic";
char const* const kQkv = "CustomQKVToContextPluginDynamic";

struct Family
{
    char const* name;
    char const* legacy;
    char const* current;
};
Family const kFamilies[] = {{kSkip, "1", "5"}, {kSkip, "2", "6"}, {kSkip, "3", "7"}, {kSkip, "4", "8"}, {kEmb, "1", "6"},
    {kEmb, "2", "4"}, {kEmb, "3", "5"}, {kQkv, "1", "4"}, {kQkv, "2", "5"}, {kQkv, "3", "6"}};

// The creator fields of one legacy version (the current version of the same family takes the same ones).
void fillFields(Fields& f, Family const& fam)
{
    std::string const v = fam.legacy;
    if (fam.name == kSkip)
    {
        int32_t const ld = 768;
        f.addFloats("beta", ld, 0.25f);
        f.addFloats("gamma", ld, 1.5f);
        if (v == "1" || v == "2")
        {
            f.addInt("type_id", 1);
            f.addFloats("bias", ld, -0.5f);
        }
        if (v == "1")
        {
            f.addInt("ld", ld);
        }
    }
    else if (fam.name == kEmb)
    {
        int32_t const ld = 128;
        f.addFloats("bert_embeddings_layernorm_beta", ld, 0.1f);
        f.addFloats("bert_embeddings_layernorm_gamma", ld, 1.1f);
        f.addFloats("bert_embeddings_word_embeddings", 50 * ld, 0.01f);
        f.addFloats("bert_embeddings_token_type_embeddings", 2 * ld, 0.02f);
        f.addFloats("bert_embeddings_position_embeddings", 64 * ld, 0.03f);
        f.addInt("output_fp16", 1);
        if (v == "1")
        {
            f.addInt("full_mask", 0);
            f.addInt("mha_type_id", 1);
        }
    }
    else if (v == "3")
    {
        f.addInt("hidden_size", 1024);
        f.addInt("num_heads", 16);
        f.addFloat("dq_probs", 1.f / 127.f);
    }
    else
    {
        f.addInt("type_id", 1);
        f.addInt("hidden_size", 768);
        f.addInt("num_heads", 12);
        f.addInt("has_mask", 1);
        if (v == "2")
        {
            f.addInt("var_seqlen", 1);
        }
    }
}

IPluginCreator* legacyCreator(Family const& fam)
{
    return static_cast<IPluginCreator*>(getPluginRegistry()->getCreator(fam.name, fam.legacy, ""));
}

IPluginCreatorV3One* currentCreator(Family const& fam)
{
    return static_cast<IPluginCreatorV3One*>(getPluginRegistry()->getCreator(fam.name, fam.current, ""));
}

// The attention plugins of legacy versions 1 and 2 serialise the runner that configurePlugin chose from the shapes, as
// the reference's do: configure them the way a builder would before asking for their stream.
template <typename Configure>
void configureIfAttention(Family const& fam, Configure configure)
{
    std::string const v = fam.legacy;
    if (fam.name != kQkv || v == "3")
    {
        return;
    }
    auto desc = [](std::initializer_list<int64_t> dims, DataType t) {
        DynamicPluginTensorDesc d{};
        d.desc.dims.nbDims = static_cast<int32_t>(dims.size());
        int i = 0;
        for (int64_t x : dims)
        {
            d.desc.dims.d[i++] = x;
        }
        d.desc.type = t;
        d.desc.format = TensorFormat::kLINEAR;
        d.desc.scale = 1.f;
        d.min = d.max = d.opt = d.desc.dims;
        return d;
    };
    if (v == "1")
    {
        DynamicPluginTensorDesc in[2] = {desc({128, 2, 3 * 768, 1, 1}, DataType::kHALF), desc({2, 512}, DataType::kINT32)};
        DynamicPluginTensorDesc out[1] = {desc({128, 2, 768, 1, 1}, DataType::kHALF)};
        configure(in, 2, out, 1);
    }
    else
    {
        DynamicPluginTensorDesc in[4] = {desc({300, 3 * 768, 1, 1}, DataType::kHALF), desc({1}, DataType::kINT32),
            desc({5}, DataType::kINT32), desc({128}, DataType::kINT32)};
        DynamicPluginTensorDesc out[1] = {desc({300, 768, 1, 1}, DataType::kHALF)};
        configure(in, 4, out, 1);
    }
}

std::vector<uint8_t> serialised(IPluginV2 const& p)
{
    std::vector<uint8_t> blob(p.getSerializationSize());
    p.serialize(blob.data());
    return blob;
}

#define CHECK(cond)                                                                                                    \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);                                                      \
            return false;                                                                                              \
        }                                                                                                              \
    } while (0)

// One pass over every family: legacy create / clone / serialise / deserialise, current create (both phases) / clone /
// field round trip.
bool exerciseAll()
{
    for (Family const& fam : kFamilies)
    {
        Fields f;
        fillFields(f, fam);
        PluginFieldCollection const* fc = f.finish();
        IPluginCreator* lc = legacyCreator(fam);
        IPluginCreatorV3One* cc = currentCreator(fam);
        CHECK(lc != nullptr && cc != nullptr);
        CHECK(lc->getFieldNames() != nullptr && cc->getFieldNames() != nullptr);
        IPluginV2* p = lc->createPlugin("layer", fc);
        CHECK(p != nullptr);
        configureIfAttention(fam, [p](DynamicPluginTensorDesc const* in, int32_t nIn, DynamicPluginTensorDesc const* out,
                                      int32_t nOut) { static_cast<IPluginV2DynamicExt*>(p)->configurePlugin(in, nIn, out, nOut); });
        std::vector<uint8_t> const blob = serialised(*p);
        CHECK(!blob.empty());
        IPluginV2* q = lc->deserializePlugin("layer", blob.data(), blob.size());
        CHECK(q != nullptr);
        CHECK(serialised(*q) == blob);
        IPluginV2* c = q->clone();
        CHECK(c != nullptr && serialised(*c) == blob);
        c->destroy();
        q->destroy();
        p->destroy();

        IPluginV3* b = cc->createPlugin("layer", fc, TensorRTPhase::kBUILD);
        CHECK(b != nullptr);
        auto* rt = static_cast<IPluginV3OneRuntime*>(b->getCapabilityInterface(PluginCapabilityType::kRUNTIME));
        CHECK(rt != nullptr);
        auto* bd = static_cast<IPluginV3OneBuild*>(b->getCapabilityInterface(PluginCapabilityType::kBUILD));
        CHECK(bd != nullptr);
        bool configured = true;
        configureIfAttention(fam, [&](DynamicPluginTensorDesc const* in, int32_t nIn, DynamicPluginTensorDesc const* out,
                                      int32_t nOut) { configured = bd->configurePlugin(in, nIn, out, nOut) == 0; });
        CHECK(configured);
        PluginFieldCollection const* ser = rt->getFieldsToSerialize();
        CHECK(ser != nullptr && ser->nbFields > 0);
        IPluginV3* r = cc->createPlugin("layer", ser, TensorRTPhase::kRUNTIME);
        CHECK(r != nullptr);
        IPluginV3* rc = r->clone();
        CHECK(rc != nullptr);
        delete rc;
        delete r;
        delete b;
    }
    return true;
}

bool runThreads()
{
    constexpr int kThreads = 8;
    constexpr int kRounds = 6;
    std::atomic<int> failures{0};
    std::vector<std::thread> pool;
    for (int t = 0; t < kThreads; ++t)
    {
        pool.emplace_back([&failures] {
            for (int i = 0; i < kRounds; ++i)
            {
                if (!exerciseAll())
                {
                    failures.fetch_add(1);
                }
            }
        });
    }
    for (auto& th : pool)
    {
        th.join();
    }
    CHECK(failures.load() == 0);
    return true;
}

// deserializePlugin on an exact-size heap copy of `bytes`; the result, if any, is used once and destroyed.
void tryStream(IPluginCreator& lc, std::vector<uint8_t> const& bytes, int& accepted, int& refused)
{
    std::unique_ptr<uint8_t[]> exact(new uint8_t[bytes.size() ? bytes.size() : 1]);
    if (!bytes.empty())
    {
        std::memcpy(exact.get(), bytes.data(), bytes.size());
    }
    IPluginV2* p = lc.deserializePlugin("fuzz", bytes.empty() ? nullptr : exact.get(), bytes.size());
    if (p != nullptr)
    {
        ++accepted;
        std::vector<uint8_t> const again = serialised(*p);
        (void) again;
        IPluginV2* c = p->clone();
        if (c != nullptr)
        {
            c->destroy();
        }
        p->destroy();
    }
    else
    {
        ++refused;
    }
}

bool runFuzz()
{
    std::mt19937 gen(20240607u);
    int accepted = 0, refused = 0, calls = 0;
    for (Family const& fam : kFamilies)
    {
        Fields f;
        fillFields(f, fam);
        IPluginCreator* lc = legacyCreator(fam);
        CHECK(lc != nullptr);
        IPluginV2* p = lc->createPlugin("layer", f.finish());
        CHECK(p != nullptr);
        configureIfAttention(fam, [p](DynamicPluginTensorDesc const* in, int32_t nIn, DynamicPluginTensorDesc const* out,
                                      int32_t nOut) { static_cast<IPluginV2DynamicExt*>(p)->configurePlugin(in, nIn, out, nOut); });
        std::vector<uint8_t> const blob = serialised(*p);
        p->destroy();
        int const before = accepted;
        tryStream(*lc, blob, accepted, refused);
        CHECK(accepted == before + 1); // the untouched stream is a plugin
        ++calls;
        // every prefix of the first 96 bytes (the scalar members), then 40 lengths spread over the rest
        std::vector<size_t> cuts;
        for (size_t n = 0; n < blob.size() && n < 96; ++n)
        {
            cuts.push_back(n);
        }
        for (int i = 0; i < 40; ++i)
        {
            cuts.push_back(gen() % blob.size());
        }
        cuts.push_back(blob.size() - 1);
        for (size_t n : cuts)
        {
            int const acc0 = accepted;
            tryStream(*lc, std::vector<uint8_t>(blob.begin(), blob.begin() + static_cast<std::ptrdiff_t>(n)), accepted, refused);
            CHECK(accepted == acc0); // a truncated stream is never a plugin
            ++calls;
        }
        // one corrupted byte among the first 64 (types, sizes, counts live there), eight values each
        for (size_t pos = 0; pos < blob.size() && pos < 64; ++pos)
        {
            for (uint8_t v : {uint8_t(0x00), uint8_t(0x01), uint8_t(0x7f), uint8_t(0x80), uint8_t(0xff)})
            {
                std::vector<uint8_t> bad = blob;
                bad[pos] = v;
                tryStream(*lc, bad, accepted, refused);
                ++calls;
            }
        }
        // huge and negative counts in every aligned 4- and 8-byte slot of the first 64 bytes
        for (size_t pos = 0; pos + 8 <= blob.size() && pos < 64; pos += 4)
        {
            for (uint64_t v : {uint64_t(0x7fffffffu), uint64_t(0xffffffffu), uint64_t(0x7fffffffffffffffull),
                     uint64_t(0xffffffffffffffffull), uint64_t(1) << 40})
            {
                std::vector<uint8_t> bad = blob;
                std::memcpy(bad.data() + pos, &v, 8);
                tryStream(*lc, bad, accepted, refused);
                ++calls;
            }
        }
        // extra bytes behind a whole stream, and random streams of the same and of small sizes
        {
            std::vector<uint8_t> longer = blob;
            longer.resize(blob.size() + 13, 0xab);
            tryStream(*lc, longer, accepted, refused);
            ++calls;
        }
        for (int i = 0; i < 24; ++i)
        {
            std::vector<uint8_t> rnd(i < 12 ? blob.size() : static_cast<size_t>(gen() % 200));
            for (auto& b : rnd)
            {
                b = static_cast<uint8_t>(gen());
            }
            tryStream(*lc, rnd, accepted, refused);
            ++calls;
        }
    }
    std::printf("fuzz: %d calls, %d accepted, %d refused\n", calls, accepted, refused);
    CHECK(calls > 1400 && refused > 1300);
    return true;
}
} // namespace

int main(int argc, char** argv)
{
    static QuietLogger logger;
    if (!initLibNvInferPlugins(&logger, ""))
    {
        std::printf("FAILED: initLibNvInferPlugins\n");
        return 1;
    }
    std::string const mode = argc > 1 ? argv[1] : "all";
    bool ok = true;
    if (mode == "threads" || mode == "all")
    {
        ok = runThreads() && ok;
    }
    if (mode == "fuzz" || mode == "all")
    {
        ok = runFuzz() && ok;
    }
    std::printf(ok ? "ok\n" : "FAILED\n");
    return ok ? 0 : 1;
}
