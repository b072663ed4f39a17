#include "Utilities/Expression/CompiledEquation.h"

#include "Utilities/Cache/LruCache.h"
#include "Utilities/Common/ScopedGpu.h"

#include <atomic>
#include <stdexcept>
#include <vector>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <mutex>

namespace ThorImplementation {

namespace {
std::atomic<uint64_t> compileCount{0};

LruCacheThreadSafe<std::string, std::shared_ptr<CompiledKernel>>& kernelCache() {
    static LruCacheThreadSafe<std::string, std::shared_ptr<CompiledKernel>> cache(10000);
    return cache;
}

LruCacheThreadSafe<std::string, std::shared_ptr<LoadedModule>>& moduleCache() {
    static LruCacheThreadSafe<std::string, std::shared_ptr<LoadedModule>> cache(10000);
    return cache;
}

std::string archOf(int deviceNum) {
    static std::mutex mutex;
    static std::vector<std::string> names;
    std::lock_guard<std::mutex> lock(mutex);
    if ((int)names.size() <= deviceNum) names.resize(deviceNum + 1);
    if (names[deviceNum].empty()) {
        thorhip_device_info info;
        THOR_HIP_CHECK(thorhip_device_get_info(deviceNum, &info));
        names[deviceNum] = info.arch_name;
    }
    return names[deviceNum];
}
}  // namespace

LoadedModule::~LoadedModule() {
    if (module != nullptr) {
        int previous = 0;
        const bool known = thorhip_get_device(&previous) == 0;
        if (known && previous != deviceNum) (void)thorhip_set_device(deviceNum);
        (void)thorhip_module_unload(module);
        if (known && previous != deviceNum) (void)thorhip_set_device(previous);
    }
}

void CompiledKernel::launch(uint32_t gridX, uint32_t gridY, uint32_t gridZ, uint32_t blockX, void* stream, std::vector<void*>& args) const {
    THOR_HIP_CHECK(thorhip_launch(function, gridX, gridY, gridZ, blockX, 1, 1, 0, stream, args.data()));
}

uint64_t compiledKernelCount() { return compileCount.load(); }

namespace {
// Every generated kernel gets a name of its own, <base>_<8 hex digits of a hash of the source>, so that profiles tell the
// kernels of different shapes apart.  All extern "C" kernels of one source share the tag.
std::string sourceTag(const std::string& source) {
    uint32_t h = 2166136261u;  // FNV-1a
    for (unsigned char ch : source) {
        h ^= ch;
        h *= 16777619u;
    }
    char text[16];
    std::snprintf(text, sizeof text, "%08x", h);
    return text;
}

std::string withTaggedKernelNames(const std::string& source, const std::string& tag) {
    static const std::string marker = "extern \"C\" __global__";
    std::string out;
    size_t pos = 0;
    while (true) {
        const size_t at = source.find(marker, pos);
        if (at == std::string::npos) break;
        const size_t paren = source.find('(', source.find(" void ", at));
        if (paren == std::string::npos) break;
        out.append(source, pos, paren - pos);
        out += "_" + tag;
        pos = paren;
    }
    out.append(source, pos, std::string::npos);
    return out;
}
}  // namespace

std::shared_ptr<CompiledKernel> compileKernel(const std::string& source, const std::string& kernelName, int deviceNum, bool fastContract) {
    const std::string moduleKey = std::to_string(deviceNum) + (fastContract ? "|contract|" : "|off|") + source;
    const std::string kernelKey = kernelName + "|" + moduleKey;
    return kernelCache().getOrCreate(kernelKey, [&] {
        ScopedGpu scoped(deviceNum);
        const std::string tag = sourceTag(source);
        const std::string taggedName = kernelName + "_" + tag;
        const std::string taggedSource = withTaggedKernelNames(source, tag);
        std::shared_ptr<LoadedModule> loaded = moduleCache().getOrCreate(moduleKey, [&] {
            const std::string arch = archOf(deviceNum);
            // "fast" contraction would also rewrite the error-compensated sequences inside the device math library (expf drops
            // from 1 ulp to ~11 ulp), so kernels that may fuse mul+add use the compiler default (fuse within an expression,
            // honour pragmas) and the others switch contraction off.
            const char* options[] = {"-ffp-contract=off"};
            const int numOptions = fastContract ? 0 : 1;
            void* code = nullptr;
            size_t codeSize = 0;
            std::vector<char> log(16384, 0);
            if (const char* dump = std::getenv("THOR_DUMP_KERNEL_SOURCE")) {
                std::ofstream out(std::string(dump) + "/" + taggedName + ".hip");
                out << taggedSource;
            }
            const int rc = thorhip_compile(taggedSource.c_str(), (taggedName + ".hip").c_str(), arch.c_str(), options, numOptions, &code, &codeSize,
                                           log.data(), log.size());
            if (rc != 0) {
                throw std::runtime_error("Run-time compilation of kernel '" + kernelName + "' failed: " + thorhip_last_error());
            }
            auto module = std::make_shared<LoadedModule>();
            module->deviceNum = deviceNum;
            const int loadRc = thorhip_module_load(&module->module, code, codeSize);
            (void)thorhip_code_free(code);
            hipCheck(loadRc, "thorhip_module_load");
            compileCount.fetch_add(1);
            return module;
        });
        auto kernel = std::make_shared<CompiledKernel>();
        kernel->module = loaded;
        kernel->deviceNum = deviceNum;
        kernel->kernelName = taggedName;
        kernel->source = taggedSource;
        THOR_HIP_CHECK(thorhip_module_get_function(&kernel->function, loaded->module, taggedName.c_str()));
        (void)thorhip_function_get_attributes(kernel->function, &kernel->numRegisters, &kernel->staticLdsBytes, nullptr);
        return kernel;
    });
}

}  // namespace ThorImplementation
