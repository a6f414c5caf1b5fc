#include "plugin_common.h"

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <mutex>
#include <set>

namespace trtamd
{
namespace plugin
{

namespace
{
std::mutex gLogMutex;
ILogger* gLogger = nullptr;
} // namespace

void setLogger(ILogger* logger)
{
    std::lock_guard<std::mutex> lock(gLogMutex);
    gLogger = logger;
}

ILogger* currentLogger()
{
    std::lock_guard<std::mutex> lock(gLogMutex);
    return gLogger;
}

void logMessage(ILogger::Severity severity, std::string const& msg)
{
    std::lock_guard<std::mutex> lock(gLogMutex);
    if (gLogger)
    {
        gLogger->log(severity, msg.c_str());
    }
    else if (severity <= ILogger::Severity::kWARNING)
    {
        std::fprintf(stderr, "[trtamd plugin] %s\n", msg.c_str());
    }
}

void reportCaught(std::exception const& e) noexcept
{
    try
    {
        logMessage(ILogger::Severity::kERROR, e.what());
    }
    catch (...)
    {
    }
}

void failValidation(char const* file, int line, char const* cond, std::string const& msg)
{
    std::ostringstream os;
    char const* base = std::strrchr(file, '/');
    os << "Validation failed: " << cond;
    if (!msg.empty())
    {
        os << " (" << msg << ")";
    }
    os << " at " << (base ? base + 1 : file) << ":" << line;
    throw PluginError(os.str());
}

int32_t getSmVersion()
{
    return 80;
}

int32_t getMHAMaskPackedSize(int32_t smVersion, DataType dataType, int32_t sequenceLength)
{
    bool const smOk = smVersion == 75 || smVersion == 80 || smVersion == 86 || smVersion == 87 || smVersion == 89
        || smVersion == 90 || smVersion == 100 || smVersion == 120;
    bool const precisionOk = dataType == DataType::kINT8 || dataType == DataType::kHALF;
    if (smOk && precisionOk)
    {
        if (sequenceLength == 64 || sequenceLength == 96 || sequenceLength == 128)
        {
            return kPackedMaskSize128;
        }
        if (sequenceLength == 384)
        {
            return kPackedMaskSize384;
        }
    }
    return kUnfusedMaskSize;
}

uint32_t getElementSize(DataType t)
{
    switch (t)
    {
    case DataType::kINT64: return 8;
    case DataType::kINT32:
    case DataType::kFLOAT: return 4;
    case DataType::kBF16:
    case DataType::kHALF: return 2;
    case DataType::kBOOL:
    case DataType::kUINT8:
    case DataType::kINT8:
    case DataType::kFP8: return 1;
    default: throw PluginError("Element size is not implemented for sub-byte data-types");
    }
}

int64_t volume(Dims const& d)
{
    int64_t v = 1;
    for (int32_t i = 0; i < d.nbDims; ++i)
    {
        v *= d.d[i];
    }
    return v;
}

DataType fieldTypeToDataType(PluginFieldType ftype)
{
    switch (ftype)
    {
    case PluginFieldType::kFLOAT32: return DataType::kFLOAT;
    case PluginFieldType::kFLOAT16: return DataType::kHALF;
    case PluginFieldType::kINT32: return DataType::kINT32;
    case PluginFieldType::kINT8: return DataType::kINT8;
    default: throw std::invalid_argument("No corresponding datatype for plugin field type");
    }
}

uint16_t floatToHalfBits(float f)
{
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint32_t const sign = (x >> 16) & 0x8000u;
    uint32_t const absx = x & 0x7fffffffu;
    if (absx > 0x7f800000u)
    {
        return static_cast<uint16_t>(sign | 0x7e00u); // NaN
    }
    if (absx >= 0x477ff000u) // >= 65520: rounds to infinity
    {
        return static_cast<uint16_t>(sign | 0x7c00u);
    }
    if (absx < 0x38800000u) // below the smallest normal binary16: quantum 2^-24
    {
        float const a = std::fabs(f);
        float const q = std::nearbyintf(a * 16777216.f);
        return static_cast<uint16_t>(sign | static_cast<uint32_t>(q));
    }
    uint32_t const mant = absx & 0x7fffffu;
    uint32_t const exp = (absx >> 23) - 112u;
    uint32_t h = (exp << 10) | (mant >> 13);
    uint32_t const rem = mant & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u)))
    {
        ++h; // a carry into the exponent is the correct rounding
    }
    return static_cast<uint16_t>(sign | h);
}

float halfBitsToFloat(uint16_t h)
{
    uint32_t const sign = static_cast<uint32_t>(h & 0x8000u) << 16;
    uint32_t const exp = (h >> 10) & 0x1fu;
    uint32_t const man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0)
    {
        float const v = static_cast<float>(man) * 5.9604644775390625e-08f;
        std::memcpy(&bits, &v, 4);
        bits |= sign;
    }
    else if (exp == 31)
    {
        bits = sign | 0x7f800000u | (man << 13);
    }
    else
    {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

void HostWeights::assign(Weights const& src, DataType type)
{
    TRTAMD_VALIDATE_MSG(type == DataType::kFLOAT || type == DataType::kHALF, "Unsupported DataType specified for plugin.");
    TRTAMD_VALIDATE_MSG(src.type == DataType::kFLOAT || src.type == DataType::kHALF,
        "weights must be binary32 or binary16");
    TRTAMD_VALIDATE(src.count >= 0);
    TRTAMD_VALIDATE(src.count == 0 || src.values != nullptr);
    mType = type;
    mCount = src.count;
    mBytes.resize(static_cast<size_t>(src.count) * getElementSize(type));
    if (src.count == 0)
    {
        return;
    }
    if (src.type == type)
    {
        std::memcpy(mBytes.data(), src.values, mBytes.size());
    }
    else if (type == DataType::kFLOAT)
    {
        auto const* s = static_cast<uint16_t const*>(src.values);
        auto* d = reinterpret_cast<float*>(mBytes.data());
        for (int64_t i = 0; i < src.count; ++i)
        {
            d[i] = halfBitsToFloat(s[i]);
        }
    }
    else
    {
        auto const* s = static_cast<float const*>(src.values);
        auto* d = reinterpret_cast<uint16_t*>(mBytes.data());
        for (int64_t i = 0; i < src.count; ++i)
        {
            d[i] = floatToHalfBits(s[i]);
        }
    }
}

bool deviceAvailable()
{
    static int const count = [] {
        int n = 0;
        if (hipGetDeviceCount(&n) != hipSuccess)
        {
            (void) hipGetLastError();
            n = 0;
        }
        return n;
    }();
    return count > 0;
}

DeviceBuffer::~DeviceBuffer()
{
    if (mPtr)
    {
        (void) hipFree(mPtr);
    }
}

void DeviceBuffer::upload(void const* host, size_t bytes)
{
    if (mPtr)
    {
        (void) hipFree(mPtr);
        mPtr = nullptr;
    }
    if (bytes == 0 || host == nullptr || !deviceAvailable())
    {
        return;
    }
    hipError_t e = hipMalloc(&mPtr, bytes);
    if (e != hipSuccess)
    {
        mPtr = nullptr;
        throw PluginError(std::string("hipMalloc failed: ") + hipGetErrorString(e));
    }
    e = hipMemcpy(mPtr, host, bytes, hipMemcpyHostToDevice);
    if (e != hipSuccess)
    {
        throw PluginError(std::string("hipMemcpy failed: ") + hipGetErrorString(e));
    }
}

void validateRequiredFields(std::initializer_list<char const*> required, PluginFieldCollection const* fc)
{
    TRTAMD_VALIDATE_MSG(fc != nullptr, "Plugin Field collection is null");
    TRTAMD_VALIDATE_MSG(fc->nbFields == 0 || fc->fields != nullptr, "Plugin Fields are null");
    std::set<std::string> missing(required.begin(), required.end());
    for (int32_t i = 0; i < fc->nbFields; ++i)
    {
        if (fc->fields[i].name)
        {
            missing.erase(fc->fields[i].name);
        }
    }
    if (!missing.empty())
    {
        std::ostringstream os;
        os << "PluginFieldCollection missing required fields: {";
        char const* sep = "";
        for (auto const& m : missing)
        {
            os << sep << m;
            sep = ", ";
        }
        os << "}";
        throw PluginError(os.str());
    }
}

PluginField const* findField(PluginFieldCollection const* fc, char const* name)
{
    if (!fc || !fc->fields)
    {
        return nullptr;
    }
    for (int32_t i = 0; i < fc->nbFields; ++i)
    {
        if (fc->fields[i].name && std::strcmp(fc->fields[i].name, name) == 0)
        {
            return &fc->fields[i];
        }
    }
    return nullptr;
}

bool readWeights(PluginFieldCollection const* fc, char const* name, Weights& out)
{
    PluginField const* f = findField(fc, name);
    if (!f)
    {
        return false;
    }
    out.type = fieldTypeToDataType(f->type);
    out.values = f->data;
    out.count = f->length;
    return true;
}

void checkKernelStatus(int status, char const* what)
{
    if (status != TRTAMD_STATUS_SUCCESS)
    {
        throw PluginError(std::string(what) + ": " + trtamd_last_error());
    }
}

} // namespace plugin
} // namespace trtamd
