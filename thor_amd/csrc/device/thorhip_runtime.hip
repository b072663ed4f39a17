// Device runtime half of the thorhip C ABI: devices, memory, streams, events, hipRTC compilation, module loading and
// kernel launch.  This is the MI355X counterpart of the function table the reference dlopen()s from the CUDA driver
// (Utilities/CudaDriver/CudaDrivertApi.h:9-158) plus its NVRTC/nvJitLink pipeline
// (Utilities/Expression/EquationCompiler.cpp:1756-1908).
#include "thorhip.h"
#include "thorhip_internal.h"
#include "thorhip_static_scratch.h"

#include <hip/hiprtc.h>

#include <atomic>
#include <cerrno>
#include <csignal>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include <dlfcn.h>
#include <poll.h>
#include <spawn.h>
#include <fcntl.h>
#include <sys/socket.h>
#include <sys/wait.h>
#include <unistd.h>

extern char** environ;

namespace thorhip {
std::string& lastError() {
    static thread_local std::string slot;
    return slot;
}
}  // namespace thorhip

using thorhip::fail;

// ---- scratch memory that exists without any allocation -----------------------------------------------------------------
// A fixed block of device memory that is part of the library's code object: every GPU the library runs on holds its own
// copy, at its own address, from the moment the code object is loaded there until the process ends.  Entry points for
// callers that must not allocate (work under stream capture, serving loops) use it where the ordinary entry points
// allocate temporary storage.  In host code the array's name is only a handle for hipGetSymbolAddress; the address that
// kernels, fills and copies use is the one looked up below, once per device, with that device current.
static __device__ __align__(256) unsigned char scratch[THORHIP_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratchMutex;
void* scratchAddress[kMaxDevices] = {};
}  // namespace

namespace thorhip {
int staticScratch(void** ptr, size_t* capacity_bytes) {
    THORHIP_REQUIRE(ptr != nullptr, "staticScratch: ptr is NULL");
    *ptr = nullptr;
    if (capacity_bytes) *capacity_bytes = THORHIP_STATIC_SCRATCH_BYTES;
    int device = -1;
    THORHIP_TRY(hipGetDevice(&device));
    THORHIP_REQUIRE(device >= 0 && device < kMaxDevices, "staticScratch: device %d is outside the table of %d devices", device, kMaxDevices);
    std::lock_guard<std::mutex> lock(scratchMutex);
    if (scratchAddress[device] == nullptr) {
        void* address = nullptr;
        THORHIP_TRY(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)));
        THORHIP_REQUIRE(address != nullptr, "staticScratch: hipGetSymbolAddress returned a null address on device %d", device);
        scratchAddress[device] = address;
    }
    *ptr = scratchAddress[device];
    return 0;
}
}  // namespace thorhip

extern "C" {

int thorhip_abi_version(void) { return THORHIP_ABI_VERSION; }

const char* thorhip_last_error(void) { return thorhip::lastError().c_str(); }

// ---- devices ---------------------------------------------------------------------------------------------------------
int thorhip_device_count(int* count) {
    THORHIP_REQUIRE(count != nullptr, "thorhip_device_count: count is NULL");
    int n = 0;
    hipError_t err = hipGetDeviceCount(&n);
    if (err == hipErrorNoDevice) {
        (void)hipGetLastError();
        *count = 0;
        return 0;
    }
    THORHIP_TRY(err);
    *count = n;
    return 0;
}

int thorhip_set_device(int device) {
    THORHIP_TRY(hipSetDevice(device));
    return 0;
}

int thorhip_get_device(int* device) {
    THORHIP_REQUIRE(device != nullptr, "thorhip_get_device: device is NULL");
    THORHIP_TRY(hipGetDevice(device));
    return 0;
}

int thorhip_device_get_info(int device, thorhip_device_info* info) {
    THORHIP_REQUIRE(info != nullptr, "thorhip_device_get_info: info is NULL");
    hipDeviceProp_t prop;
    THORHIP_TRY(hipGetDeviceProperties(&prop, device));
    std::memset(info, 0, sizeof *info);
    info->compute_units = prop.multiProcessorCount;
    info->wavefront_size = prop.warpSize;
    info->max_threads_per_block = prop.maxThreadsPerBlock;
    info->lds_bytes_per_block = (int)prop.sharedMemPerBlock;
    info->l2_bytes = prop.l2CacheSize;
    info->clock_khz = prop.clockRate;
    info->memory_clock_khz = prop.memoryClockRate;
    info->memory_bus_width_bits = prop.memoryBusWidth;
    info->total_global_mem = prop.totalGlobalMem;
    std::snprintf(info->arch_name, sizeof info->arch_name, "%s", prop.gcnArchName);
    std::snprintf(info->name, sizeof info->name, "%s", prop.name);
    return 0;
}

int thorhip_device_synchronize(void) {
    THORHIP_TRY(hipDeviceSynchronize());
    return 0;
}

// ---- memory ----------------------------------------------------------------------------------------------------------
int thorhip_malloc(void** ptr, size_t bytes) {
    THORHIP_REQUIRE(ptr != nullptr, "thorhip_malloc: ptr is NULL");
    *ptr = nullptr;
    if (bytes == 0) return 0;
    hipError_t err = hipMalloc(ptr, bytes);
    if (err != hipSuccess) {
        size_t free_b = 0, total_b = 0;
        (void)hipMemGetInfo(&free_b, &total_b);
        (void)hipGetLastError();
        return fail(-(int)err - 1000, "hipMalloc(%zu bytes) failed: %s; device memory free %zu of %zu bytes", bytes,
                    hipGetErrorName(err), free_b, total_b);
    }
    return 0;
}

int thorhip_free(void* ptr) {
    if (ptr == nullptr) return 0;
    THORHIP_TRY(hipFree(ptr));
    return 0;
}

int thorhip_host_malloc(void** ptr, size_t bytes) {
    THORHIP_REQUIRE(ptr != nullptr, "thorhip_host_malloc: ptr is NULL");
    *ptr = nullptr;
    if (bytes == 0) return 0;
    THORHIP_TRY(hipHostMalloc(ptr, bytes, hipHostMallocDefault));
    return 0;
}

int thorhip_host_free(void* ptr) {
    if (ptr == nullptr) return 0;
    THORHIP_TRY(hipHostFree(ptr));
    return 0;
}

int thorhip_memcpy_async(void* dst, const void* src, size_t bytes, int kind, void* stream) {
    if (bytes == 0) return 0;
    THORHIP_REQUIRE(dst != nullptr && src != nullptr, "thorhip_memcpy_async: NULL pointer");
    hipMemcpyKind k;
    switch (kind) {
        case THORHIP_H2D:
            k = hipMemcpyHostToDevice;
            break;
        case THORHIP_D2H:
            k = hipMemcpyDeviceToHost;
            break;
        case THORHIP_D2D:
            k = hipMemcpyDeviceToDevice;
            break;
        default:
            return fail(-1, "thorhip_memcpy_async: unknown copy kind %d", kind);
    }
    THORHIP_TRY(hipMemcpyAsync(dst, src, bytes, k, (hipStream_t)stream));
    return 0;
}

int thorhip_memset_async(void* dst, int byte_value, size_t bytes, void* stream) {
    if (bytes == 0) return 0;
    THORHIP_REQUIRE(dst != nullptr, "thorhip_memset_async: dst is NULL");
    THORHIP_TRY(hipMemsetAsync(dst, byte_value, bytes, (hipStream_t)stream));
    return 0;
}

int thorhip_mem_get_info(size_t* free_bytes, size_t* total_bytes) {
    size_t f = 0, t = 0;
    THORHIP_TRY(hipMemGetInfo(&f, &t));
    if (free_bytes) *free_bytes = f;
    if (total_bytes) *total_bytes = t;
    return 0;
}

// ---- streams / events ------------------------------------------------------------------------------------------------
int thorhip_stream_create(void** stream) {
    THORHIP_REQUIRE(stream != nullptr, "thorhip_stream_create: stream is NULL");
    hipStream_t s = nullptr;
    THORHIP_TRY(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = s;
    return 0;
}

int thorhip_stream_destroy(void* stream) {
    if (stream == nullptr) return 0;
    THORHIP_TRY(hipStreamDestroy((hipStream_t)stream));
    return 0;
}

int thorhip_stream_synchronize(void* stream) {
    THORHIP_TRY(hipStreamSynchronize((hipStream_t)stream));
    return 0;
}

int thorhip_stream_wait_event(void* stream, void* event) {
    THORHIP_REQUIRE(event != nullptr, "thorhip_stream_wait_event: event is NULL");
    THORHIP_TRY(hipStreamWaitEvent((hipStream_t)stream, (hipEvent_t)event, 0));
    return 0;
}

int thorhip_stream_enqueue_host_function(void* stream, thorhip_host_fn fn, void* user_data) {
    THORHIP_REQUIRE(fn != nullptr, "thorhip_stream_enqueue_host_function: fn is NULL");
    THORHIP_TRY(hipLaunchHostFunc((hipStream_t)stream, fn, user_data));
    return 0;
}

int thorhip_event_create(void** event, int enable_timing) {
    THORHIP_REQUIRE(event != nullptr, "thorhip_event_create: event is NULL");
    hipEvent_t e = nullptr;
    THORHIP_TRY(hipEventCreateWithFlags(&e, enable_timing ? hipEventDefault : hipEventDisableTiming));
    *event = e;
    return 0;
}

int thorhip_event_destroy(void* event) {
    if (event == nullptr) return 0;
    THORHIP_TRY(hipEventDestroy((hipEvent_t)event));
    return 0;
}

int thorhip_event_record(void* event, void* stream) {
    THORHIP_REQUIRE(event != nullptr, "thorhip_event_record: event is NULL");
    THORHIP_TRY(hipEventRecord((hipEvent_t)event, (hipStream_t)stream));
    return 0;
}

int thorhip_event_synchronize(void* event) {
    THORHIP_REQUIRE(event != nullptr, "thorhip_event_synchronize: event is NULL");
    THORHIP_TRY(hipEventSynchronize((hipEvent_t)event));
    return 0;
}

int thorhip_event_elapsed_ms(float* ms, void* start, void* stop) {
    THORHIP_REQUIRE(ms != nullptr && start != nullptr && stop != nullptr, "thorhip_event_elapsed_ms: NULL argument");
    THORHIP_TRY(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return 0;
}

// ---- run-time compilation ---------------------------------------------------------------------------------------------
static void copyLog(hiprtcProgram prog, char* log, size_t cap) {
    if (log == nullptr || cap == 0) return;
    log[0] = '\0';
    size_t n = 0;
    if (hiprtcGetProgramLogSize(prog, &n) != HIPRTC_SUCCESS || n == 0) return;
    std::string text(n, '\0');
    if (hiprtcGetProgramLog(prog, text.data()) != HIPRTC_SUCCESS) return;
    std::snprintf(log, cap, "%s", text.c_str());
}

// ---- compilation in a process of its own ------------------------------------------------------------------------------
// -1: not decided yet (THORHIP_COMPILE_ISOLATION in the environment decides at the first compile), 0 off, 1 on
static std::atomic<int> compileIsolation{-1};

static bool isolationEnabled() {
    int mode = compileIsolation.load();
    if (mode < 0) {
        const char* env = std::getenv("THORHIP_COMPILE_ISOLATION");
        mode = (env != nullptr && std::atoi(env) != 0) ? 1 : 0;
        compileIsolation.store(mode);
    }
    return mode == 1;
}

// The worker sits next to this library (built by the same Makefile); THORHIP_RTC_WORKER names another one.
static std::string workerPath() {
    if (const char* env = std::getenv("THORHIP_RTC_WORKER")) return env;
    Dl_info info;
    if (dladdr(reinterpret_cast<const void*>(&thorhip_abi_version), &info) != 0 && info.dli_fname != nullptr) {
        std::string path = info.dli_fname;
        const size_t slash = path.rfind('/');
        return (slash == std::string::npos ? std::string(".") : path.substr(0, slash)) + "/thorhip_rtc_worker";
    }
    return "thorhip_rtc_worker";
}

static bool sendAll(int fd, const void* data, size_t bytes) {
    const char* p = static_cast<const char*>(data);
    while (bytes > 0) {
        const ssize_t n = ::send(fd, p, bytes, MSG_NOSIGNAL);  // a worker that died must not raise SIGPIPE here
        if (n < 0 && errno == EINTR) continue;
        if (n <= 0) return false;
        p += n;
        bytes -= static_cast<size_t>(n);
    }
    return true;
}
static bool sendString(int fd, const std::string& s) {
    const uint64_t n = s.size();
    return sendAll(fd, &n, sizeof n) && (n == 0 || sendAll(fd, s.data(), n));
}

// Runs one compilation in the worker program.  The worker gets the request on its standard input and answers on its standard
// output; what it (or the compiler inside it) prints to standard error is kept for the error text.  A worker that ends on a
// signal - the compiler called abort() - is reported as a failed compilation; the calling process is never replaced or harmed.
static int compileInWorker(const std::string& source, const std::string& name, const std::string& arch, const std::vector<std::string>& flags,
                           void** code, size_t* code_size, char* log, size_t log_capacity) {
    const std::string path = workerPath();
    // Every descriptor is close-on-exec from its creation, so a worker started by another thread at the same moment inherits none
    // of them (it would hold this call's pipes open and keep its reader waiting for an end that never comes); the three the
    // worker needs are duplicated onto its standard descriptors, which clears the flag on the copies.
    int toWorker[2] = {-1, -1}, fromWorker[2] = {-1, -1}, errWorker[2] = {-1, -1};
    auto closeAll = [&] {
        for (int* pair : {toWorker, fromWorker, errWorker})
            for (int k = 0; k < 2; ++k)
                if (pair[k] >= 0) ::close(pair[k]);
    };
    if (socketpair(AF_UNIX, SOCK_STREAM | SOCK_CLOEXEC, 0, toWorker) != 0) return fail(-7, "thorhip_compile: socketpair failed: %s", std::strerror(errno));
    if (pipe2(fromWorker, O_CLOEXEC) != 0 || pipe2(errWorker, O_CLOEXEC) != 0) {
        const int reason = errno;
        closeAll();
        return fail(-7, "thorhip_compile: pipe failed: %s", std::strerror(reason));
    }
    // a process that runs with closed standard descriptors may have been handed 0, 1 or 2 here: duplicating a descriptor onto itself
    // would leave its close-on-exec flag set, so the worker's ends are moved out of that range first
    for (int* end : {&toWorker[0], &fromWorker[1], &errWorker[1]}) {
        if (*end > STDERR_FILENO) continue;
        const int moved = fcntl(*end, F_DUPFD_CLOEXEC, STDERR_FILENO + 1);
        if (moved < 0) {
            const int reason = errno;
            closeAll();
            return fail(-7, "thorhip_compile: cannot move a descriptor: %s", std::strerror(reason));
        }
        ::close(*end);
        *end = moved;
    }
    posix_spawn_file_actions_t actions;
    posix_spawn_file_actions_init(&actions);
    posix_spawn_file_actions_adddup2(&actions, toWorker[0], STDIN_FILENO);
    posix_spawn_file_actions_adddup2(&actions, fromWorker[1], STDOUT_FILENO);
    posix_spawn_file_actions_adddup2(&actions, errWorker[1], STDERR_FILENO);
    char* const argv[] = {const_cast<char*>(path.c_str()), nullptr};
    pid_t pid = -1;
    const int spawned = posix_spawn(&pid, path.c_str(), &actions, nullptr, argv, environ);
    posix_spawn_file_actions_destroy(&actions);
    ::close(toWorker[0]);
    ::close(fromWorker[1]);
    ::close(errWorker[1]);
    if (spawned != 0) {
        for (int fd : {toWorker[1], fromWorker[0], errWorker[0]}) ::close(fd);
        return fail(-7, "thorhip_compile: cannot start the compiler worker '%s': %s", path.c_str(), std::strerror(spawned));
    }
    bool sent = sendString(toWorker[1], name) && sendString(toWorker[1], arch) && sendString(toWorker[1], source);
    const uint64_t optionCount = flags.size();
    sent = sent && sendAll(toWorker[1], &optionCount, sizeof optionCount);
    for (const std::string& f : flags) sent = sent && sendString(toWorker[1], f);
    ::close(toWorker[1]);

    std::string answer, errors;
    pollfd fds[2] = {{fromWorker[0], POLLIN, 0}, {errWorker[0], POLLIN, 0}};
    int open = 2;
    while (open > 0) {
        if (poll(fds, 2, -1) < 0) {
            if (errno == EINTR) continue;
            break;
        }
        for (int i = 0; i < 2; ++i) {
            if (fds[i].fd < 0 || (fds[i].revents & (POLLIN | POLLHUP | POLLERR)) == 0) continue;
            char buffer[65536];
            const ssize_t n = ::read(fds[i].fd, buffer, sizeof buffer);
            if (n > 0) {
                (i == 0 ? answer : errors).append(buffer, static_cast<size_t>(n));
            } else if (n == 0 || errno != EINTR) {
                ::close(fds[i].fd);
                fds[i].fd = -1;
                --open;
            }
        }
    }
    for (pollfd& f : fds)
        if (f.fd >= 0) ::close(f.fd);
    int status = 0;
    while (waitpid(pid, &status, 0) < 0 && errno == EINTR) {
    }
    if (errors.size() > 1500) errors = errors.substr(0, 700) + "\n...\n" + errors.substr(errors.size() - 700);
    if (WIFSIGNALED(status)) {
        return fail(-8, "thorhip_compile: the compiler ended on signal %d (%s) while compiling '%s' for %s; the calling process is unharmed.\n%s",
                    WTERMSIG(status), strsignal(WTERMSIG(status)), name.c_str(), arch.c_str(), errors.c_str());
    }
    if (!sent) return fail(-8, "thorhip_compile: the compiler worker closed its input early (exit status %d).\n%s", WEXITSTATUS(status), errors.c_str());
    // answer: status, code (length, bytes), log (length, bytes)
    auto take = [&](size_t& at, void* into, size_t bytes) {
        if (answer.size() < at + bytes) return false;
        std::memcpy(into, answer.data() + at, bytes);
        at += bytes;
        return true;
    };
    size_t at = 0;
    int64_t workerStatus = 0;
    uint64_t codeBytes = 0, logBytes = 0;
    if (!take(at, &workerStatus, sizeof workerStatus) || !take(at, &codeBytes, sizeof codeBytes) || answer.size() < at + codeBytes) {
        return fail(-8, "thorhip_compile: the compiler worker gave no complete answer (exit status %d).\n%s", WEXITSTATUS(status), errors.c_str());
    }
    const size_t codeAt = at;
    at += codeBytes;
    std::string workerLog;
    if (take(at, &logBytes, sizeof logBytes) && answer.size() >= at + logBytes) workerLog.assign(answer, at, logBytes);
    if (log != nullptr && log_capacity > 0) std::snprintf(log, log_capacity, "%s", workerLog.c_str());
    if (workerStatus != 0 || codeBytes == 0) return fail(-3, "hiprtcCompileProgram(%s) failed in the compiler worker: %s", arch.c_str(), workerLog.c_str());
    void* blob = std::malloc(codeBytes);
    if (blob == nullptr) return fail(-5, "thorhip_compile: out of host memory for a %zu byte code object", (size_t)codeBytes);
    std::memcpy(blob, answer.data() + codeAt, codeBytes);
    *code = blob;
    *code_size = codeBytes;
    return 0;
}

int thorhip_set_compile_isolation(int enabled) {
    const int before = isolationEnabled() ? 1 : 0;
    compileIsolation.store(enabled != 0 ? 1 : 0);
    return before;
}

int thorhip_compile(const char* source, const char* program_name, const char* arch, const char* const* options,
                    int num_options, void** code, size_t* code_size, char* log, size_t log_capacity) {
    THORHIP_REQUIRE(source != nullptr && code != nullptr && code_size != nullptr, "thorhip_compile: NULL argument");
    *code = nullptr;
    *code_size = 0;
    if (log && log_capacity) log[0] = '\0';

    std::string arch_name;
    if (arch != nullptr && arch[0] != '\0') {
        arch_name = arch;
    } else {
        int dev = 0;
        hipDeviceProp_t prop;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.gcnArchName[0]) {
            arch_name = prop.gcnArchName;
        } else {
            (void)hipGetLastError();
            arch_name = "gfx950";
        }
    }
    const std::string arch_flag = "--offload-arch=" + arch_name;

    if (isolationEnabled()) {
        std::vector<std::string> workerFlags = {arch_flag, "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
        for (int i = 0; i < num_options; ++i) workerFlags.push_back(options[i]);
        return compileInWorker(source, program_name ? program_name : "thor_fused.hip", arch_name, workerFlags, code, code_size, log, log_capacity);
    }

    hiprtcProgram prog = nullptr;
    hiprtcResult rc = hiprtcCreateProgram(&prog, source, program_name ? program_name : "thor_fused.hip", 0, nullptr, nullptr);
    if (rc != HIPRTC_SUCCESS) return fail(-2, "hiprtcCreateProgram failed: %s", hiprtcGetErrorString(rc));

    // Fixed flags: gfx950 code object, wave64 (the gfx9 default), -O3, and the packed-fp32 VALU forms switched off.
    std::vector<const char*> flags = {arch_flag.c_str(), "-O3",    "-std=c++17",     "-Xclang",
                                      "-target-feature", "-Xclang", "-packed-fp32-ops"};
    for (int i = 0; i < num_options; ++i) flags.push_back(options[i]);

    rc = hiprtcCompileProgram(prog, (int)flags.size(), flags.data());
    copyLog(prog, log, log_capacity);
    if (rc != HIPRTC_SUCCESS) {
        std::string text;
        size_t n = 0;
        if (hiprtcGetProgramLogSize(prog, &n) == HIPRTC_SUCCESS && n > 0) {
            text.resize(n);
            (void)hiprtcGetProgramLog(prog, text.data());
        }
        (void)hiprtcDestroyProgram(&prog);
        return fail(-3, "hiprtcCompileProgram(%s) failed: %s\n%s", arch_name.c_str(), hiprtcGetErrorString(rc), text.c_str());
    }
    size_t n = 0;
    rc = hiprtcGetCodeSize(prog, &n);
    if (rc != HIPRTC_SUCCESS || n == 0) {
        (void)hiprtcDestroyProgram(&prog);
        return fail(-4, "hiprtcGetCodeSize failed: %s", hiprtcGetErrorString(rc));
    }
    void* blob = std::malloc(n);
    if (blob == nullptr) {
        (void)hiprtcDestroyProgram(&prog);
        return fail(-5, "thorhip_compile: out of host memory for a %zu byte code object", n);
    }
    rc = hiprtcGetCode(prog, (char*)blob);
    (void)hiprtcDestroyProgram(&prog);
    if (rc != HIPRTC_SUCCESS) {
        std::free(blob);
        return fail(-6, "hiprtcGetCode failed: %s", hiprtcGetErrorString(rc));
    }
    *code = blob;
    *code_size = n;
    return 0;
}

int thorhip_code_free(void* code) {
    std::free(code);
    return 0;
}

int thorhip_module_load(void** module, const void* code, size_t code_size) {
    THORHIP_REQUIRE(module != nullptr && code != nullptr && code_size > 0, "thorhip_module_load: bad argument");
    hipModule_t m = nullptr;
    THORHIP_TRY(hipModuleLoadData(&m, code));
    *module = m;
    return 0;
}

int thorhip_module_unload(void* module) {
    if (module == nullptr) return 0;
    THORHIP_TRY(hipModuleUnload((hipModule_t)module));
    return 0;
}

int thorhip_module_get_function(void** function, void* module, const char* kernel_name) {
    THORHIP_REQUIRE(function != nullptr && module != nullptr && kernel_name != nullptr, "thorhip_module_get_function: NULL argument");
    hipFunction_t f = nullptr;
    THORHIP_TRY(hipModuleGetFunction(&f, (hipModule_t)module, kernel_name));
    *function = f;
    return 0;
}

int thorhip_function_get_attributes(void* function, int* num_vgprs_hint, int* static_lds_bytes, int* max_threads_per_block) {
    THORHIP_REQUIRE(function != nullptr, "thorhip_function_get_attributes: function is NULL");
    int v = 0;
    if (num_vgprs_hint) {
        THORHIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, (hipFunction_t)function));
        *num_vgprs_hint = v;
    }
    if (static_lds_bytes) {
        THORHIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_SHARED_SIZE_BYTES, (hipFunction_t)function));
        *static_lds_bytes = v;
    }
    if (max_threads_per_block) {
        THORHIP_TRY(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_MAX_THREADS_PER_BLOCK, (hipFunction_t)function));
        *max_threads_per_block = v;
    }
    return 0;
}

int thorhip_launch(void* function, uint32_t grid_x, uint32_t grid_y, uint32_t grid_z, uint32_t block_x, uint32_t block_y,
                   uint32_t block_z, uint32_t dynamic_lds_bytes, void* stream, void** args) {
    THORHIP_REQUIRE(function != nullptr, "thorhip_launch: function is NULL");
    THORHIP_REQUIRE(grid_x > 0 && grid_y > 0 && grid_z > 0 && block_x > 0 && block_y > 0 && block_z > 0,
                    "thorhip_launch: empty grid or block (%u,%u,%u)x(%u,%u,%u)", grid_x, grid_y, grid_z, block_x, block_y, block_z);
    THORHIP_REQUIRE((uint64_t)block_x * block_y * block_z <= 1024, "thorhip_launch: block of %llu threads exceeds 1024",
                    (unsigned long long)block_x * block_y * block_z);
    THORHIP_TRY(hipModuleLaunchKernel((hipFunction_t)function, grid_x, grid_y, grid_z, block_x, block_y, block_z,
                                      dynamic_lds_bytes, (hipStream_t)stream, args, nullptr));
    return 0;
}

}  // extern "C"
