// Compiler worker of the thorhip C ABI: one run-time compilation in a process of its own.
//
// thorhip_compile starts this program when compile isolation is on, so that a compiler that aborts (an internal compiler error
// ends in abort(), which would take the caller's process down with it) only ends this process.  The worker links the run-time
// compiler alone and makes no device call: it never touches a GPU.
//
// Protocol, all on stdin / stdout, integers as native 64-bit words:
//   request : program name, architecture, source (each: length, bytes), option count, options (each: length, bytes)
//   response: status (0 success, else the hiprtcResult or a negative worker error), code object (length, bytes), log (length, bytes)
#include <hip/hiprtc.h>

#include <cstdint>
#include <cstdio>
#include <string>
#include <unistd.h>
#include <vector>

namespace {
bool readAll(void* into, size_t bytes) {
    char* p = static_cast<char*>(into);
    while (bytes > 0) {
        const ssize_t n = ::read(STDIN_FILENO, p, bytes);
        if (n <= 0) return false;
        p += n;
        bytes -= static_cast<size_t>(n);
    }
    return true;
}
bool writeAll(const void* from, size_t bytes) {
    const char* p = static_cast<const char*>(from);
    while (bytes > 0) {
        const ssize_t n = ::write(STDOUT_FILENO, p, bytes);
        if (n <= 0) return false;
        p += n;
        bytes -= static_cast<size_t>(n);
    }
    return true;
}
bool readString(std::string& s) {
    uint64_t n = 0;
    if (!readAll(&n, sizeof n) || n > (1ull << 30)) return false;
    s.resize(n);
    return n == 0 || readAll(s.data(), n);
}
bool writeBlob(const std::string& s) {
    const uint64_t n = s.size();
    return writeAll(&n, sizeof n) && (n == 0 || writeAll(s.data(), n));
}
int respond(int64_t status, const std::string& code, const std::string& log) {
    return writeAll(&status, sizeof status) && writeBlob(code) && writeBlob(log) ? 0 : 3;
}
}  // namespace

int main() {
    std::string name, arch, source;
    uint64_t optionCount = 0;
    if (!readString(name) || !readString(arch) || !readString(source) || !readAll(&optionCount, sizeof optionCount) || optionCount > 256) return 2;
    std::vector<std::string> options(optionCount);
    for (std::string& o : options)
        if (!readString(o)) return 2;

    hiprtcProgram program = nullptr;
    hiprtcResult rc = hiprtcCreateProgram(&program, source.c_str(), name.c_str(), 0, nullptr, nullptr);
    if (rc != HIPRTC_SUCCESS) return respond(rc, "", std::string("hiprtcCreateProgram failed: ") + hiprtcGetErrorString(rc));
    std::vector<const char*> flags;
    for (const std::string& o : options) flags.push_back(o.c_str());
    rc = hiprtcCompileProgram(program, static_cast<int>(flags.size()), flags.data());
    std::string log;
    size_t logSize = 0;
    if (hiprtcGetProgramLogSize(program, &logSize) == HIPRTC_SUCCESS && logSize > 0) {
        log.resize(logSize);
        if (hiprtcGetProgramLog(program, log.data()) != HIPRTC_SUCCESS) log.clear();
    }
    if (rc != HIPRTC_SUCCESS) {
        (void)hiprtcDestroyProgram(&program);
        return respond(rc, "", std::string("hiprtcCompileProgram failed: ") + hiprtcGetErrorString(rc) + "\n" + log);
    }
    size_t codeSize = 0;
    std::string code;
    rc = hiprtcGetCodeSize(program, &codeSize);
    if (rc == HIPRTC_SUCCESS && codeSize > 0) {
        code.resize(codeSize);
        rc = hiprtcGetCode(program, code.data());
    }
    (void)hiprtcDestroyProgram(&program);
    if (rc != HIPRTC_SUCCESS || code.empty()) return respond(rc == HIPRTC_SUCCESS ? -4 : rc, "", "hiprtcGetCode failed");
    return respond(0, code, log);
}
