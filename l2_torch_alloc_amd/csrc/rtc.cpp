#include "rtc.h"

#include <elf.h>
#include <hip/hip_version.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <atomic>
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

// True when every #include of the text names one of the in-memory compatibility headers or a
// header below hip/ : files whose content is fixed by the ROCm installation, which the cache key
// identifies.  Any other include (in either spelling, with any spacing) may change under the key.
bool includes_only_toolchain_headers(const std::string& source) {
    size_t pos = 0;
    while ((pos = source.find('#', pos)) != std::string::npos) {
        // a directive starts its line (blanks aside); a '#' anywhere else is text
        size_t line = pos;
        while (line > 0 && (source[line - 1] == ' ' || source[line - 1] == '\t')) line--;
        const bool directive = line == 0 || source[line - 1] == '\n';
        size_t p = pos + 1;
        pos = p;
        if (!directive) continue;
        while (p < source.size() && (source[p] == ' ' || source[p] == '\t')) p++;
        if (source.compare(p, 7, "include") != 0) continue;
        p += 7;
        while (p < source.size() && (source[p] == ' ' || source[p] == '\t')) p++;
        if (p >= source.size() || (source[p] != '"' && source[p] != '<')) return false;    // a macro-built name
        const char close = source[p] == '"' ? '"' : '>';
        const size_t end = source.find(close, p + 1);
        if (end == std::string::npos) return false;
        const std::string name = source.substr(p + 1, end - p - 1);
        bool known = name.compare(0, 4, "hip/") == 0;
        for (const char* compat : kCompatNames) known = known || name == compat;
        if (!known) return false;
    }
    return true;
}

// Names the compiler and its headers: the hipRTC version, the HIP version this library was built
// against, and the version file of the ROCm installation the headers come from.
std::string toolchain_identity() {
    int maj = 0, min = 0;
    hiprtcVersion(&maj, &min);
    std::string id = "hiprtc " + std::to_string(maj) + "." + std::to_string(min) + " hip " +
                     std::to_string(HIP_VERSION_MAJOR) + "." + std::to_string(HIP_VERSION_MINOR) + "." +
                     std::to_string(HIP_VERSION_PATCH) + " rocm ";
    std::ifstream f(rocm_root() + "/.info/version");
    std::string line;
    if (f && std::getline(f, line)) id += line;
    return id;
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
    // a name of its own per writer: two threads of one process may compile the same text at once
    static std::atomic<unsigned long> serial{0};
    std::string tmp = path + ".tmp" + std::to_string((long)::getpid()) + "_" + std::to_string(serial.fetch_add(1));
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

size_t read_code_object_symbol(const std::vector<char>& code, const char* name, void* out, size_t capacity) {
    const size_t size = code.size();
    const char* base = code.data();
    if (size < sizeof(Elf64_Ehdr) || std::memcmp(base, ELFMAG, SELFMAG) != 0 || base[EI_CLASS] != ELFCLASS64) return 0;
    Elf64_Ehdr eh;
    std::memcpy(&eh, base, sizeof eh);
    if (eh.e_shentsize != sizeof(Elf64_Shdr) || eh.e_shoff > size ||
        (size - eh.e_shoff) / sizeof(Elf64_Shdr) < eh.e_shnum) return 0;
    auto section = [&](unsigned i, Elf64_Shdr* sh) {
        if (i >= eh.e_shnum) return false;
        std::memcpy(sh, base + eh.e_shoff + (size_t)i * sizeof(Elf64_Shdr), sizeof *sh);
        return sh->sh_type == SHT_NOBITS || (sh->sh_offset <= size && sh->sh_size <= size - sh->sh_offset);
    };
    const size_t name_len = std::strlen(name);
    for (unsigned i = 0; i < eh.e_shnum; i++) {
        Elf64_Shdr symtab, strtab;
        if (!section(i, &symtab) || (symtab.sh_type != SHT_SYMTAB && symtab.sh_type != SHT_DYNSYM)) continue;
        if (symtab.sh_entsize != sizeof(Elf64_Sym) || !section(symtab.sh_link, &strtab) || strtab.sh_type != SHT_STRTAB) continue;
        for (size_t k = 0; k < symtab.sh_size / sizeof(Elf64_Sym); k++) {
            Elf64_Sym sym;
            std::memcpy(&sym, base + symtab.sh_offset + k * sizeof sym, sizeof sym);
            if (sym.st_name >= strtab.sh_size || strtab.sh_size - sym.st_name <= name_len) continue;
            const char* s = base + strtab.sh_offset + sym.st_name;
            if (std::memcmp(s, name, name_len) != 0 || s[name_len] != '\0') continue;
            Elf64_Shdr data;
            if (sym.st_shndx == SHN_UNDEF || sym.st_shndx >= SHN_LORESERVE || !section(sym.st_shndx, &data) ||
                data.sh_type == SHT_NOBITS || sym.st_value < data.sh_addr) continue;
            const uint64_t off = sym.st_value - data.sh_addr;
            if (off > data.sh_size) continue;
            size_t n = sym.st_size < capacity ? (size_t)sym.st_size : capacity;
            if (n > data.sh_size - off) n = (size_t)(data.sh_size - off);
            std::memcpy(out, base + data.sh_offset + off, n);
            return n;
        }
    }
    return 0;
}

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
        // The first kernel arguments (the launch plan's scalars, then the i0 and o0 pointers and the
        // feedback word's: as many as fit in fourteen registers) are handed to every wave in registers at its start
        // instead of being fetched by its first instructions.  With one workgroup per 4 KiB chunk
        // that fetch is on the critical path of every workgroup: 16 MiB copies run 8 % faster
        // with the preload, 64 MiB copies 3 %.  The code object keeps a prologue that fetches the
        // same arguments for firmware that does not preload.
        "-mllvm", "-amdgpu-kernarg-preload-count=11",
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
    // Sources that include anything but the ROCm headers are not cached (the content of a user's
    // file is not in the key).
    std::string dir = includes_only_toolchain_headers(source) ? cache_dir() : "";
    std::string cache_path;
    if (!dir.empty()) {
        uint64_t h = fnv1a(source);
        for (auto& o : opts) h = fnv1a(o, h);
        h = fnv1a(toolchain_identity(), h);
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
