// A kernel compiled at run time for one GPU: the loaded code object, the kernel function handle and its launch shape.
// Shared through a process-wide LRU keyed by the generated source text, so equal stages compile once
// (reference: Utilities/Expression/CompiledEquation.h:96-103 owns the CUmodule the same way;
//  Utilities/Expression/EquationCompiler.cpp:1916-1988 keeps the global kernel cache).
#pragma once

#include "DeepLearning/Implementation/Tensor/Tensor.h"

#include <cstdint>
#include <memory>
#include <string>
#include <vector>

namespace ThorImplementation {

// A scalar that lives in device memory: one element of `sourceDType` at `byteOffset` inside `buffer`, read by the kernels at
// every run, so a stamped plan follows a value that other GPU work updates (reference: CompiledEquation.h:15-19 there).
struct TensorScalarBinding {
    Tensor buffer;
    uint64_t byteOffset = 0;
    DataType sourceDType = DataType::FP32;
};

// A loaded code object; unloaded when the last kernel handle that refers to it goes away (errors are swallowed).
struct LoadedModule {
    LoadedModule() = default;
    LoadedModule(const LoadedModule&) = delete;
    LoadedModule& operator=(const LoadedModule&) = delete;
    ~LoadedModule();
    void* module = nullptr;
    int deviceNum = 0;
    std::shared_ptr<const std::string> source;  // the compiled text, one copy for every kernel of the module
};

struct CompiledKernel {
    std::shared_ptr<LoadedModule> module;
    void* function = nullptr;
    int deviceNum = 0;
    std::string kernelName;
    // the text the module was compiled from (diagnostics and tests)
    const std::string& source() const {
        static const std::string none;
        return module && module->source ? *module->source : none;
    }
    int numRegisters = 0;
    int staticLdsBytes = 0;

    // Asynchronous launch on `stream` (a raw stream handle of the same GPU).
    void launch(uint32_t gridX, uint32_t gridY, uint32_t gridZ, uint32_t blockX, void* stream, std::vector<void*>& args) const;
};

// Compiles (or fetches from the process-wide cache) `kernelName` from `source` for GPU `deviceNum`.  `fastContract`
// keeps the compiler's default contraction (a*b+c inside one expression may fuse, matching the reference's
// -fmad=true); false compiles with -ffp-contract=off so every operation rounds on its own.
std::shared_ptr<CompiledKernel> compileKernel(const std::string& source, const std::string& kernelName, int deviceNum, bool fastContract);

// The cached kernel, or null when `compileKernel` has not built it in this process (nothing is compiled or loaded).
std::shared_ptr<CompiledKernel> findLoadedKernel(const std::string& source, const std::string& kernelName, int deviceNum, bool fastContract);

// Number of run-time compilations performed so far (cache misses); used by tests of the caching behaviour.
uint64_t compiledKernelCount();

}  // namespace ThorImplementation
