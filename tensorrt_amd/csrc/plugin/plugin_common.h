// Shared host-side machinery of the BERT plugin classes: logging, the error convention, host
// weights with binary16/binary32 conversion, device-resident parameters and PluginField parsing.
//
// Conventions follow the reference plugin library: every interface method is noexcept, wraps its
// body in try/catch, logs through the registered ILogger and returns a failure value
// (plugin/common/plugin.h:34-41, plugin/vc/checkMacrosPlugin.h:58-282).  Unlike the reference's
// PLUGIN_ASSERT, nothing here resets the device or exits the process: a violated precondition
// throws and the calling interface method reports failure.
#pragma once

#include "trtamd_bert_kernels.h"
#include "trtamd_nvinfer_api.h"

#include <cstdint>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace trtamd
{
namespace plugin
{

using namespace nvinfer1;

// pluginStatus_t of the reference
enum PluginStatus : int32_t
{
    kSTATUS_SUCCESS = 0,
    kSTATUS_FAILURE = 1,
    kSTATUS_BAD_PARAM = 2,
    kSTATUS_NOT_SUPPORTED = 3,
    kSTATUS_NOT_INITIALIZED = 4
};

// Index of the sequence, batch and hidden dimensions of [S,B,E,1,1] tensors (plugin/common/bertCommon.h:55-57).
constexpr int32_t kSDIM = 0;
constexpr int32_t kBDIM = 1;
constexpr int32_t kHDIM = 2;

// Packed-mask sizes per sequence (plugin/common/bertCommon.h:68-84).
constexpr int32_t kUnfusedMaskSize = 1;
constexpr int32_t kPackedMaskSize128 = 4 * (2 * 2 * 32);   // S in {64, 96, 128}
constexpr int32_t kPackedMaskSize384 = 24 * (1 * 8 * 32);  // S = 384

// ---- logging -----------------------------------------------------------------------------------

void setLogger(ILogger* logger);
ILogger* currentLogger();
void logMessage(ILogger::Severity severity, std::string const& msg);

class PluginError : public std::runtime_error
{
public:
    explicit PluginError(std::string const& what)
        : std::runtime_error(what)
    {
    }
};

// Logs an exception caught at an interface boundary (caughtError of the reference).
void reportCaught(std::exception const& e) noexcept;

[[noreturn]] void failValidation(char const* file, int line, char const* cond, std::string const& msg);

#define TRTAMD_VALIDATE(cond)                                                                                          \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            ::trtamd::plugin::failValidation(__FILE__, __LINE__, #cond, std::string());                                \
        }                                                                                                              \
    } while (0)

#define TRTAMD_VALIDATE_MSG(cond, msg)                                                                                 \
    do                                                                                                                 \
    {                                                                                                                  \
        if (!(cond))                                                                                                   \
        {                                                                                                              \
            ::trtamd::plugin::failValidation(__FILE__, __LINE__, #cond, (msg));                                        \
        }                                                                                                              \
    } while (0)

// ---- small helpers -----------------------------------------------------------------------------

// Capability class reported where the reference reports the CUDA SM version: the fused attention
// kernels of this library cover what the reference has on SM 8.0 and later.
int32_t getSmVersion();

// getMHAMaskPackedSize (plugin/common/bertCommon.h:114-140).
int32_t getMHAMaskPackedSize(int32_t smVersion, DataType dataType, int32_t sequenceLength);

// getElementSize (plugin/common/bertCommon.h:142-160).
uint32_t getElementSize(DataType t);

int64_t volume(Dims const& d);

// fieldTypeToDataType (plugin/common/bertCommon.h:507-533).
DataType fieldTypeToDataType(PluginFieldType ftype);

uint16_t floatToHalfBits(float f);
float halfBitsToFloat(uint16_t h);

// ---- weights -----------------------------------------------------------------------------------

// Host copy of a weight tensor in a chosen type (binary32 or binary16), converted with
// round-to-nearest-even like WeightsWithOwnership::convertAndCopy (plugin/common/bertCommon.h:358-445).
class HostWeights
{
public:
    HostWeights() = default;
    void assign(Weights const& src, DataType type);
    Weights view() const
    {
        return Weights{mType, mBytes.empty() ? nullptr : mBytes.data(), mCount};
    }
    bool empty() const
    {
        return mCount == 0;
    }
    int64_t count() const
    {
        return mCount;
    }
    DataType type() const
    {
        return mType;
    }
    void const* data() const
    {
        return mBytes.data();
    }
    size_t bytes() const
    {
        return mBytes.size();
    }

private:
    DataType mType{DataType::kFLOAT};
    int64_t mCount{0};
    std::vector<uint8_t> mBytes;
};

// Device copy of host bytes (copyToDevice, plugin/common/bertCommon.h:447-457).  Uploaded when a
// plugin is constructed if a GPU is present; on a machine without one (host-only tests) the buffer
// stays empty and enqueue reports the plugin as not initialised.
class DeviceBuffer
{
public:
    DeviceBuffer() = default;
    ~DeviceBuffer();
    DeviceBuffer(DeviceBuffer const&) = delete;
    DeviceBuffer& operator=(DeviceBuffer const&) = delete;
    void upload(void const* host, size_t bytes);
    void upload(HostWeights const& w)
    {
        upload(w.data(), w.bytes());
    }
    void* get() const
    {
        return mPtr;
    }
    template <typename T>
    T const* as() const
    {
        return static_cast<T const*>(mPtr);
    }

private:
    void* mPtr{nullptr};
};

bool deviceAvailable();

// ---- PluginField parsing -----------------------------------------------------------------------

// validateRequiredAttributesExist (plugin/common/plugin.cpp:135-155): throws with
// "PluginFieldCollection missing required fields: {a, b}".
void validateRequiredFields(std::initializer_list<char const*> required, PluginFieldCollection const* fc);

PluginField const* findField(PluginFieldCollection const* fc, char const* name);

// Weight-valued field as a Weights view (type from the field type).
bool readWeights(PluginFieldCollection const* fc, char const* name, Weights& out);

template <typename T>
bool readScalar(PluginFieldCollection const* fc, char const* name, T& out)
{
    PluginField const* f = findField(fc, name);
    if (!f || !f->data)
    {
        return false;
    }
    std::memcpy(&out, f->data, sizeof(T));
    return true;
}

// Owns the PluginField array a plugin hands out from getFieldsToSerialize().
class FieldList
{
public:
    void clear()
    {
        mFields.clear();
    }
    void add(char const* name, void const* data, PluginFieldType type, int32_t length)
    {
        mFields.emplace_back(name, data, type, length);
    }
    PluginFieldCollection const* collection()
    {
        mFC.nbFields = static_cast<int32_t>(mFields.size());
        mFC.fields = mFields.data();
        return &mFC;
    }

private:
    std::vector<PluginField> mFields;
    PluginFieldCollection mFC{};
};

// Turns a C-ABI status into an exception carrying trtamd_last_error().
void checkKernelStatus(int status, char const* what);

} // namespace plugin
} // namespace trtamd
