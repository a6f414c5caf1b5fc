// Stand-alone plugin registry and the library's exported C entry points.
//
// On a machine with TensorRT the closed-source libnvinfer implements getPluginRegistry() and the
// plugin library's static PluginRegistrar objects register into it at load time
// (include/NvInferRuntime.h:5044, 5092-5109; e.g. plugin/skipLayerNormPlugin/skipLayerNormPlugin.cpp:41-42).
// There is no libnvinfer for MI355X, so this library ships the registry itself: creators are kept
// by (namespace, name, version) and looked up with getCreator(name, version, ns), exactly what an
// engine-side caller does (samples/sampleNonZeroPlugin/sampleNonZeroPlugin.cpp:509-515).
#include "plugin_base.h"

#include <dlfcn.h>

#include <map>
#include <mutex>
#include <tuple>

namespace trtamd
{
namespace plugin
{
namespace
{

class Registry final : public IPluginRegistry
{
public:
    void setErrorRecorder(IErrorRecorder* const recorder) noexcept override
    {
        mRecorder = recorder;
    }
    IErrorRecorder* getErrorRecorder() const noexcept override
    {
        return mRecorder;
    }
    bool isParentSearchEnabled() const override
    {
        return mParentSearch;
    }
    void setParentSearchEnabled(bool const enabled) override
    {
        mParentSearch = enabled;
    }

    // Loads a plugin library and registers what its getCreators() returns
    // (plugin/vc/vfcCommon.cpp:68-79 is the library side of this protocol).
    PluginLibraryHandle loadLibrary(AsciiChar const* pluginPath) noexcept override
    {
        try
        {
            TRTAMD_VALIDATE(pluginPath != nullptr);
            void* handle = dlopen(pluginPath, RTLD_LAZY | RTLD_LOCAL);
            TRTAMD_VALIDATE_MSG(handle != nullptr, std::string("dlopen failed: ") + dlerror());
            using GetCreatorsFn = IPluginCreatorInterface* const* (*) (int32_t&);
            using SetLoggerFinderFn = void (*)(ILoggerFinder*);
            auto setFinder = reinterpret_cast<SetLoggerFinderFn>(dlsym(handle, "setLoggerFinder"));
            auto getCreatorsFn = reinterpret_cast<GetCreatorsFn>(dlsym(handle, "getCreators"));
            if (!getCreatorsFn)
            {
                dlclose(handle);
                throw PluginError("library exports no getCreators()");
            }
            (void) setFinder;
            int32_t n = 0;
            IPluginCreatorInterface* const* creators = getCreatorsFn(n);
            std::lock_guard<std::mutex> lock(mMutex);
            for (int32_t i = 0; i < n; ++i)
            {
                addLocked(*creators[i], "", handle);
            }
            return handle;
        }
        catch (std::exception const& e)
        {
            reportCaught(e);
        }
        return nullptr;
    }

    void deregisterLibrary(PluginLibraryHandle handle) noexcept override
    {
        std::lock_guard<std::mutex> lock(mMutex);
        for (auto it = mCreators.begin(); it != mCreators.end();)
        {
            it = it->second.library == handle && handle != nullptr ? mCreators.erase(it) : std::next(it);
        }
        rebuildListLocked();
    }

    bool registerCreator(IPluginCreatorInterface& creator, AsciiChar const* const pluginNamespace) noexcept override
    {
        try
        {
            std::lock_guard<std::mutex> lock(mMutex);
            return addLocked(creator, pluginNamespace ? pluginNamespace : "", nullptr);
        }
        catch (std::exception const& e)
        {
            reportCaught(e);
        }
        return false;
    }

    IPluginCreatorInterface* const* getAllCreators(int32_t* const numCreators) const noexcept override
    {
        std::lock_guard<std::mutex> lock(mMutex);
        if (numCreators)
        {
            *numCreators = static_cast<int32_t>(mList.size());
        }
        return mList.empty() ? nullptr : mList.data();
    }

    IPluginCreatorInterface* getCreator(AsciiChar const* const pluginName, AsciiChar const* const pluginVersion,
        AsciiChar const* const pluginNamespace) noexcept override
    {
        if (!pluginName || !pluginVersion)
        {
            return nullptr;
        }
        std::lock_guard<std::mutex> lock(mMutex);
        auto it = mCreators.find(Key{pluginNamespace ? pluginNamespace : "", pluginName, pluginVersion});
        return it == mCreators.end() ? nullptr : it->second.creator;
    }

    bool deregisterCreator(IPluginCreatorInterface const& creator) noexcept override
    {
        std::lock_guard<std::mutex> lock(mMutex);
        for (auto it = mCreators.begin(); it != mCreators.end(); ++it)
        {
            if (it->second.creator == &creator)
            {
                mCreators.erase(it);
                rebuildListLocked();
                return true;
            }
        }
        return false;
    }

    IPluginResource* acquirePluginResource(AsciiChar const* key, IPluginResource* resource) noexcept override
    {
        try
        {
            if (!key || !resource)
            {
                return nullptr;
            }
            std::lock_guard<std::mutex> lock(mMutex);
            auto& slot = mResources[key];
            if (slot.count == 0)
            {
                slot.resource = resource->clone();
            }
            if (!slot.resource)
            {
                mResources.erase(key);
                return nullptr;
            }
            ++slot.count;
            return slot.resource;
        }
        catch (std::exception const& e)
        {
            reportCaught(e);
        }
        return nullptr;
    }

    int32_t releasePluginResource(AsciiChar const* key) noexcept override
    {
        if (!key)
        {
            return -1;
        }
        std::lock_guard<std::mutex> lock(mMutex);
        auto it = mResources.find(key);
        if (it == mResources.end())
        {
            return -1;
        }
        if (--it->second.count == 0)
        {
            it->second.resource->release();
            mResources.erase(it);
        }
        return 0;
    }

    IPluginCreatorInterface* const* getAllCreatorsRecursive(int32_t* const numCreators) noexcept override
    {
        return getAllCreators(numCreators);
    }

private:
    using Key = std::tuple<std::string, std::string, std::string>;
    struct Entry
    {
        IPluginCreatorInterface* creator;
        void* library;
    };
    struct Resource
    {
        IPluginResource* resource{nullptr};
        int32_t count{0};
    };

    bool addLocked(IPluginCreatorInterface& creator, std::string const& ns, void* library)
    {
        // IPluginCreatorV3One and the deprecated IPluginCreator carry a name and a version to key on
        InterfaceInfo const info = creator.getInterfaceInfo();
        std::string const kind = info.kind ? info.kind : "";
        char const* name = nullptr;
        char const* version = nullptr;
        if (kind == "PLUGIN CREATOR_V3ONE")
        {
            auto& c = static_cast<IPluginCreatorV3One&>(creator);
            name = c.getPluginName();
            version = c.getPluginVersion();
        }
        else if (kind == "PLUGIN CREATOR_V1")
        {
            auto& c = static_cast<IPluginCreator&>(creator);
            name = c.getPluginName();
            version = c.getPluginVersion();
        }
        if (!name || !version)
        {
            logMessage(ILogger::Severity::kERROR, "registerCreator: unsupported creator interface");
            return false;
        }
        Key key{ns, name, version};
        if (mCreators.count(key))
        {
            logMessage(ILogger::Severity::kVERBOSE,
                std::string("Plugin creator already registered - ") + name + " version " + version);
            return false;
        }
        mCreators.emplace(std::move(key), Entry{&creator, library});
        rebuildListLocked();
        return true;
    }

    void rebuildListLocked()
    {
        mList.clear();
        for (auto const& kv : mCreators)
        {
            mList.push_back(kv.second.creator);
        }
    }

    mutable std::mutex mMutex;
    std::map<Key, Entry> mCreators;
    std::vector<IPluginCreatorInterface*> mList;
    std::map<std::string, Resource> mResources;
    IErrorRecorder* mRecorder{nullptr};
    bool mParentSearch{true};
};

} // namespace
} // namespace plugin
} // namespace trtamd

using namespace trtamd::plugin;

extern "C" nvinfer1::IPluginRegistry* getPluginRegistry() noexcept
{
    // function-local static: constructed on first use, i.e. by the first static PluginRegistrar
    static Registry* registry = new Registry();
    return registry;
}

extern "C" nvinfer1::ILogger* getLogger() noexcept
{
    return currentLogger();
}

extern "C" bool initLibNvInferPlugins(void* logger, char const* /*libNamespace*/)
{
    // The BERT creators register themselves when the library is loaded (static registrars); this
    // call only installs the logger and is safe to repeat (plugin/api/inferPlugin.cpp:171-209).
    if (logger)
    {
        setLogger(static_cast<nvinfer1::ILogger*>(logger));
    }
    return true;
}

extern "C" void setLoggerFinder(nvinfer1::ILoggerFinder* finder)
{
    if (finder && !currentLogger())
    {
        setLogger(finder->findLogger());
    }
}

extern "C" nvinfer1::IPluginCreatorInterface* const* getCreators(int32_t& nbCreators)
{
    auto const& list = recordedCreators();
    nbCreators = static_cast<int32_t>(list.size());
    return list.data();
}
