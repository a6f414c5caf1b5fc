// An engine-side caller written against the plugin interface alone (compiled by g++, no HIP headers): looks the
// three BERT plugins up in the registry by the reference's names and versions, creates them from
// PluginFieldCollections, walks their capability interfaces and round-trips one through its serialised fields.
// Prints "ok" and returns 0 when every check holds.  Nothing here launches a kernel.
#include "trtamd_nvinfer_api.h"

#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

using namespace nvinfer1;

#define CHECK(cond)                                                                                                    \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            std::printf("FAILED line %d: %s\n", __LINE__, #cond);                                                      \
            return 1;                                                                                                  \
        }                                                                                                              \
    } while (0)

namespace
{
class QuietLogger final : public ILogger
{
public:
    void log(Severity severity, AsciiChar const* msg) noexcept override
    {
        if (severity <= Severity::kERROR)
        {
            last = msg ? msg : "";
        }
    }
    std::string last;
};

IPluginCreatorV3One* creatorOf(char const* name, char const* version)
{
    return static_cast<IPluginCreatorV3One*>(getPluginRegistry()->getCreator(name, version, ""));
}
} // namespace

int main()
{
    QuietLogger logger;
    CHECK(initLibNvInferPlugins(&logger, ""));

    // every current version of the three plugins is there, under the reference's names
    char const* const skip = "CustomSkipLayerNormPluginDynamic";
    char const* const emb = "CustomEmbLayerNormPluginDynamic";
    char const* const qkv = "CustomQKVToContextPluginDynamic";
    for (char const* v : {"5", "6", "7", "8"})
    {
        CHECK(creatorOf(skip, v) != nullptr);
    }
    for (char const* v : {"4", "5", "6"})
    {
        CHECK(creatorOf(emb, v) != nullptr);
        CHECK(creatorOf(qkv, v) != nullptr);
    }
    CHECK(creatorOf(skip, "99") == nullptr);
    int32_t nbCreators = 0;
    CHECK(getPluginRegistry()->getAllCreators(&nbCreators) != nullptr && nbCreators >= 20);

    // SkipLayerNorm version 6, FP16, with bias
    constexpr int32_t ld = 768;
    std::vector<float> beta(ld, 0.25f), gamma(ld, 1.5f), bias(ld, -0.5f);
    int32_t const typeId = static_cast<int32_t>(DataType::kHALF);
    std::vector<PluginField> fields{{"type_id", &typeId, PluginFieldType::kINT32, 1},
        {"beta", beta.data(), PluginFieldType::kFLOAT32, ld}, {"gamma", gamma.data(), PluginFieldType::kFLOAT32, ld},
        {"bias", bias.data(), PluginFieldType::kFLOAT32, ld}};
    PluginFieldCollection fc{static_cast<int32_t>(fields.size()), fields.data()};
    IPluginCreatorV3One* creator = creatorOf(skip, "6");
    CHECK(std::strcmp(creator->getPluginName(), skip) == 0 && std::strcmp(creator->getPluginVersion(), "6") == 0);
    PluginFieldCollection const* advertised = creator->getFieldNames();
    CHECK(advertised != nullptr && advertised->nbFields == 4);

    IPluginV3* plugin = creator->createPlugin("skipln", &fc, TensorRTPhase::kBUILD);
    CHECK(plugin != nullptr);
    auto* core = static_cast<IPluginV3OneCore*>(plugin->getCapabilityInterface(PluginCapabilityType::kCORE));
    auto* build = static_cast<IPluginV3OneBuild*>(plugin->getCapabilityInterface(PluginCapabilityType::kBUILD));
    auto* runtime = static_cast<IPluginV3OneRuntime*>(plugin->getCapabilityInterface(PluginCapabilityType::kRUNTIME));
    CHECK(core && build && runtime);
    CHECK(std::strcmp(core->getPluginName(), skip) == 0 && std::strcmp(core->getPluginVersion(), "6") == 0);
    CHECK(build->getNbOutputs() == 1);
    DataType const inTypes[2] = {DataType::kHALF, DataType::kHALF};
    DataType outType = DataType::kFLOAT;
    CHECK(build->getOutputDataTypes(&outType, 1, inTypes, 2) == 0 && outType == DataType::kHALF);

    DynamicPluginTensorDesc io[3]{};
    for (auto& d : io)
    {
        d.desc.dims.nbDims = 5;
        int64_t const shape[5] = {128, 4, ld, 1, 1};
        std::memcpy(d.desc.dims.d, shape, sizeof(shape));
        d.desc.type = DataType::kHALF;
        d.desc.format = TensorFormat::kLINEAR;
        d.desc.scale = 1.f;
        d.min = d.max = d.opt = d.desc.dims;
    }
    for (int32_t pos = 0; pos < 3; ++pos)
    {
        CHECK(build->supportsFormatCombination(pos, io, 2, 1));
    }
    io[0].desc.type = DataType::kFLOAT;
    CHECK(!build->supportsFormatCombination(0, io, 2, 1));
    io[0].desc.type = DataType::kHALF;
    CHECK(build->configurePlugin(io, 2, io + 2, 1) == 0);
    CHECK(build->getWorkspaceSize(io, 2, io + 2, 1) == 0);

    // what an engine file holds, and the plugin rebuilt from it
    PluginFieldCollection const* serialised = runtime->getFieldsToSerialize();
    CHECK(serialised != nullptr && serialised->nbFields >= 3);
    IPluginV3* rebuilt = creator->createPlugin("skipln", serialised, TensorRTPhase::kRUNTIME);
    CHECK(rebuilt != nullptr);
    IPluginV3* copy = rebuilt->clone();
    CHECK(copy != nullptr);
    auto* copyRuntime = static_cast<IPluginV3OneRuntime*>(copy->getCapabilityInterface(PluginCapabilityType::kRUNTIME));
    PluginFieldCollection const* again = copyRuntime->getFieldsToSerialize();
    CHECK(again != nullptr && again->nbFields == serialised->nbFields);
    for (int32_t i = 0; i < again->nbFields; ++i)
    {
        CHECK(std::strcmp(again->fields[i].name, serialised->fields[i].name) == 0);
        CHECK(again->fields[i].length == serialised->fields[i].length && again->fields[i].type == serialised->fields[i].type);
    }

    // a missing required field is refused and the reason is logged
    logger.last.clear();
    PluginFieldCollection incomplete{2, fields.data()};
    CHECK(creator->createPlugin("bad", &incomplete, TensorRTPhase::kBUILD) == nullptr);
    CHECK(!logger.last.empty());

    delete copy;
    delete rebuilt;
    delete plugin;
    std::printf("ok\n");
    return 0;
}
