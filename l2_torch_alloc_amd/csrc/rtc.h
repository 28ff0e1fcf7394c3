// Run-time compilation of kernel source for gfx950 with hipRTC, and the small services around
// it: in-memory compatibility headers, an on-disk cache of code objects, and an ISA dump.
// Takes the place of the reference's NVRTC -> cubin step (sideaware.cu:523-607).
#pragma once

#include <string>
#include <vector>

namespace sideaware {

struct CompileResult {
    bool ok = false;
    bool from_disk_cache = false;
    std::vector<char> code;     // gfx950 code object
    std::string log;            // compiler diagnostics (warnings on success, errors on failure)
};

// Compiles `source` (one translation unit, already holding the configuration block, the user's
// header and the kernel template).  Needs no GPU: hipRTC cross-compiles.  `use_disk_cache` false
// compiles afresh and overwrites whatever the cache holds for this source (the way out when a
// cached code object turns out not to load).
CompileResult compile_for_gfx950(const std::string& source, const char* arch = "gfx950",
                                 bool use_disk_cache = true);

// Copies the initial bytes of a global variable out of a code object (an ELF image), on the host:
// what a kernel says about itself (tile size, entry point name) is known without asking the
// device, so a first-use compile neither copies from the device nor waits for it.  Returns the
// number of bytes copied (at most `capacity`), 0 if the symbol is not there.
size_t read_code_object_symbol(const std::vector<char>& code, const char* name, void* out, size_t capacity);

// Where every later successful compile appends its disassembly ("" = nowhere).  The reference
// dumps SASS through cuobjdump (sideaware.cu:572-599); here it is the gfx950 ISA of the code
// object just built, through the ROCm llvm-objdump.
void set_isa_dump_file(const std::string& filename);

}  // namespace sideaware
