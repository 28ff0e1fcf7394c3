#include "rtc.h"

#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <fstream>
#include <mutex>

namespace sideaware {

namespace {

std::mutex g_rtc_mu;
std::string g_isa_file;

// User op headers written for the reference pull in CUDA's fp16/bf16 headers by name and use
// CUDA's spelling of the bf16 type (test.py:192-198).  These in-memory headers give hipRTC
// files of those names that only forward to the HIP headers and add the one alias; nothing of
// the CUDA runtime is emulated.
const char* kCompatNames[] = {"cuda_fp16.h", "cuda_bf16.h", "cuda_runtime.h"};
const char* kCompatBodies[] = {
    "#pragma once\n#include <hip/hip_fp16.h>\n",
    "#pragma once\n#include <hip/hip_bf16.h>\ntypedef __hip_bfloat16 __nv_bfloat16;\n"
    "typedef __hip_bfloat162 __nv_bfloat162;\n",
    "#pragma once\n",
};

std::string rocm_root() {
    const char* env = std::getenv("ROCM_PATH");
    return env && *env ? env : "/opt/rocm";
}

uint64_t fnv1a(const std::string& s, uint64_t h = 1469598103934665603ull) {
    for (unsigned char c : s) { h ^= c; h *= 1099511628211ull; }
    return h;
}

uint64_t fnv1a(const std::vector<char>& v) {
    uint64_t h = 1469598103934665603ull;
    for (char c : v) { h ^= (unsigned char)c; h *= 1099511628211ull; }
    return h;
}

std::string cache_dir() {
    if (const char* off = std::getenv("SIDEAWARE_NO_DISK_CACHE")) {
        if (*off && *off != '0') return "";
    }
    std::string dir;
    if (const char* d = std::getenv("SIDEAWARE_CACHE_DIR")) dir = d;
    else if (const char* x = std::getenv("XDG_CACHE_HOME")) dir = std::string(x) + "/sideaware_gfx950";
    else if (const char* h = std::getenv("HOME")) dir = std::string(h) + "/.cache/sideaware_gfx950";
    if (dir.empty()) return "";
    ::mkdir(dir.substr(0, dir.find_last_of('/')).c_str(), 0755);
    ::mkdir(dir.c_str(), 0755);
    return ::access(dir.c_str(), W_OK) == 0 ? dir : "";
}

bool read_file(const std::string& path, std::vector<char>& out) {
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) return false;
    std::streamsize n = f.tellg();
    if (n <= 0) return false;
    out.resize((size_t)n);
    f.seekg(0);
    return (bool)f.read(out.data(), n);
}

void write_file_atomic(const std::string& path, const std::vector<char>& data) {
    std::string tmp = path + ".tmp" + std::to_string((long)::getpid());
    {
        std::ofstream f(tmp, std::ios::binary);
        if (!f) return;
        f.write(data.data(), (std::streamsize)data.size());
        if (!f) { ::unlink(tmp.c_str()); return; }
    }
    if (::rename(tmp.c_str(), path.c_str()) != 0) ::unlink(tmp.c_str());
}

// A cache file is the code object followed by the eight bytes of its FNV-1a hash: a file that was
// cut short or damaged reads as a miss instead of reaching the module loader.
bool read_cached_code(const std::string& path, std::vector<char>& code) {
    std::vector<char> raw;
    if (!read_file(path, raw) || raw.size() <= 8 + 4) return false;
    uint64_t stored = 0;
    std::memcpy(&stored, raw.data() + raw.size() - 8, 8);
    raw.resize(raw.size() - 8);
    if (fnv1a(raw) != stored || std::memcmp(raw.data(), "\177ELF", 4) != 0) return false;
    code.swap(raw);
    return true;
}

void write_cached_code(const std::string& path, const std::vector<char>& code) {
    std::vector<char> raw(code);
    const uint64_t h = fnv1a(code);
    raw.insert(raw.end(), (const char*)&h, (const char*)&h + 8);
    write_file_atomic(path, raw);
}

void dump_isa(const std::vector<char>& code) {
    std::string file;
    {
        std::lock_guard<std::mutex> g(g_rtc_mu);
        file = g_isa_file;
    }
    if (file.empty()) return;
    char tmpl[] = "/tmp/sideaware_co_XXXXXX";
    int fd = ::mkstemp(tmpl);
    if (fd < 0) return;
    ssize_t w = ::write(fd, code.data(), code.size());
    ::close(fd);
    if (w == (ssize_t)code.size()) {
        std::string cmd = rocm_root() + "/lib/llvm/bin/llvm-objdump -d --no-show-raw-insn " + tmpl + " 2>/dev/null";
        if (FILE* pipe = ::popen(cmd.c_str(), "r")) {
            std::ofstream out(file, std::ios::app);
            char stamp[64];
            std::time_t now = std::time(nullptr);
            std::strftime(stamp, sizeof stamp, "%F %T", std::localtime(&now));
            out << "==================== gfx950 ISA (" << stamp << ") ====================\n";
            char buf[4096];
            while (std::fgets(buf, sizeof buf, pipe)) out << buf;
            out << "==================== end ====================\n";
            ::pclose(pipe);
        }
    }
    ::unlink(tmpl);
}

}  // namespace

void set_isa_dump_file(const std::string& filename) {
    std::lock_guard<std::mutex> g(g_rtc_mu);
    g_isa_file = filename;
}

CompileResult compile_for_gfx950(const std::string& source, const char* arch, bool use_disk_cache) {
    CompileResult res;

    char cwd_buf[4096];
    std::string cwd = ::getcwd(cwd_buf, sizeof cwd_buf) ? cwd_buf : ".";
    std::vector<std::string> opts = {
        std::string("--offload-arch=") + arch,
        "-O3",
        "-std=c++17",
        // Products are rounded before they are added: results match a CPU that does not fuse,
        // bit for bit.  An op header that wants fused math can say so with a pragma.
        "-ffp-contract=off",
        // The compiler is kept from forming packed fp32 instructions out of scalar code.
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-I" + rocm_root() + "/include",
        "-I" + cwd,                       // op headers may #include "file" relative to the cwd
        "-Wno-unused-parameter",
    };
    if (const char* extra = std::getenv("SIDEAWARE_RTC_FLAGS")) {
        std::string e(extra);
        size_t pos = 0;
        while (pos < e.size()) {
            size_t sp = e.find(' ', pos);
            if (sp == std::string::npos) sp = e.size();
            if (sp > pos) opts.push_back(e.substr(pos, sp - pos));
            pos = sp + 1;
        }
    }

    // Disk cache: the key covers the whole translation unit, every option and the compiler.
    // Sources that include files by path are not cached (their content is not in the key).
    std::string dir = source.find("#include \"") == std::string::npos ? cache_dir() : "";
    std::string cache_path;
    if (!dir.empty()) {
        int maj = 0, min = 0;
        hiprtcVersion(&maj, &min);
        uint64_t h = fnv1a(source);
        for (auto& o : opts) h = fnv1a(o, h);
        h = fnv1a(std::to_string(maj) + "." + std::to_string(min), h);
        char name[64];
        std::snprintf(name, sizeof name, "/%016llx.co", (unsigned long long)h);
        cache_path = dir + name;
        if (use_disk_cache && read_cached_code(cache_path, res.code)) {
            res.ok = true;
            res.from_disk_cache = true;
            dump_isa(res.code);
            return res;
        }
    }

    std::vector<const char*> copts;
    for (auto& o : opts) copts.push_back(o.c_str());

    // One compile at a time: callers compile different ops from different threads, and nothing
    // promises that the compiler library underneath tolerates that.
    static std::mutex compile_mu;
    std::lock_guard<std::mutex> compile_guard(compile_mu);

    hiprtcProgram prog = nullptr;
    hiprtcResult rc = hiprtcCreateProgram(&prog, source.c_str(), "sideaware_elementwise.hip",
                                          (int)(sizeof kCompatNames / sizeof *kCompatNames),
                                          kCompatBodies, kCompatNames);
    if (rc != HIPRTC_SUCCESS) {
        res.log = std::string("hiprtcCreateProgram: ") + hiprtcGetErrorString(rc);
        return res;
    }
    rc = hiprtcCompileProgram(prog, (int)copts.size(), copts.data());
    size_t log_size = 0;
    if (hiprtcGetProgramLogSize(prog, &log_size) == HIPRTC_SUCCESS && log_size > 1) {
        res.log.resize(log_size);
        hiprtcGetProgramLog(prog, &res.log[0]);
        while (!res.log.empty() && res.log.back() == '\0') res.log.pop_back();
    }
    if (rc != HIPRTC_SUCCESS) {
        res.log += std::string("\nhiprtcCompileProgram: ") + hiprtcGetErrorString(rc);
        hiprtcDestroyProgram(&prog);
        return res;
    }
    size_t code_size = 0;
    if (hiprtcGetCodeSize(prog, &code_size) != HIPRTC_SUCCESS || code_size == 0) {
        res.log += "\nhiprtcGetCodeSize failed";
        hiprtcDestroyProgram(&prog);
        return res;
    }
    res.code.resize(code_size);
    rc = hiprtcGetCode(prog, res.code.data());
    hiprtcDestroyProgram(&prog);
    if (rc != HIPRTC_SUCCESS) {
        res.log += std::string("\nhiprtcGetCode: ") + hiprtcGetErrorString(rc);
        res.code.clear();
        return res;
    }
    res.ok = true;
    if (!cache_path.empty()) write_cached_code(cache_path, res.code);
    dump_isa(res.code);
    return res;
}

}  // namespace sideaware
