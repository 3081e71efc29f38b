#include "hip_kernel.hpp"

#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <sstream>

#include "HipRuntime.hpp"

namespace acro
{

namespace
{

const char *const kCompileOptions[] = {
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
};
constexpr int kNumCompileOptions = sizeof(kCompileOptions) / sizeof(kCompileOptions[0]);

// The two experiment hooks below replace what the library compiles, so they are only honoured when
// ACRO_HIP_DEBUG_HOOKS=1 says that this is wanted.
bool debugHooks()
{
    const char *env = std::getenv("ACRO_HIP_DEBUG_HOOKS");
    return env != nullptr && std::string(env) == "1";
}

// Experiment hook: further options for the run-time compiler, separated by blanks (ACRO_HIP_COMPILE_OPTIONS="-mllvm
// -amdgpu-..."); they are part of the key of the on-disk cache.
std::vector<std::string> extraCompileOptions()
{
    std::vector<std::string> extra;
    const char *env = debugHooks() ? std::getenv("ACRO_HIP_COMPILE_OPTIONS") : nullptr;
    if (env == nullptr) return extra;
    std::istringstream words(env);
    std::string word;
    while (words >> word) extra.push_back(word);
    return extra;
}

uint64_t fnv1a(const std::string &s, uint64_t h = 1469598103934665603ull)
{
    for (unsigned char c : s)
    {
        h ^= c;
        h *= 1099511628211ull;
    }
    return h;
}

std::string cacheDir()
{
    const char *env = std::getenv("ACRO_HIP_CACHE_DIR");
    if (env != nullptr)
    {
        if (std::string(env) == "off" || std::string(env).empty()) return "";
        return env;
    }
    const char *home = std::getenv("HOME");
    if (home == nullptr || *home == '\0') return "";
    return std::string(home) + "/.cache/acrotensor_hip";
}

bool makeDirs(const std::string &path)
{
    std::string partial;
    for (size_t i = 0; i <= path.size(); ++i)
    {
        if (i == path.size() || path[i] == '/')
        {
            if (!partial.empty() && ::mkdir(partial.c_str(), 0755) != 0 && errno != EEXIST) return false;
        }
        if (i < path.size()) partial += path[i];
    }
    return true;
}

std::string cachePath(const std::string &name, const std::string &source)
{
    std::string dir = cacheDir();
    if (dir.empty()) return "";
    int major = 0, minor = 0;
    hiprtcVersion(&major, &minor);
    std::string salt = std::to_string(major) + "." + std::to_string(minor);
    for (int i = 0; i < kNumCompileOptions; ++i) salt += std::string(" ") + kCompileOptions[i];
    for (const std::string &option : extraCompileOptions()) salt += " " + option;
    uint64_t h = fnv1a(source, fnv1a(salt + name));
    char hex[32];
    std::snprintf(hex, sizeof(hex), "%016llx", static_cast<unsigned long long>(h));
    return dir + "/" + hex + ".hsaco";
}

void rtcCheck(hiprtcResult r, const char *what)
{
    if (r != HIPRTC_SUCCESS)
    {
        throw_error(std::string("hipRTC failure in ") + what + ": " + hiprtcGetErrorString(r));
    }
}

}  // namespace

// The code object is an ELF file (64-bit, little endian) in which every kernel has a 64-byte descriptor under the
// symbol "<name>.kd"; bytes 4 - 7 of the descriptor are private_segment_fixed_size.  hipRTC may wrap the ELF file in
// a bundle ("__CLANG_OFFLOAD_BUNDLE__"): the first ELF file inside it is taken (there is one target).
int HipKernel::PrivateSegmentBytes(const std::vector<char> &code_object, const std::string &function)
{
    const unsigned char *base = reinterpret_cast<const unsigned char *>(code_object.data());
    size_t size = code_object.size();
    auto rd = [&](size_t at, int bytes) -> uint64_t {
        uint64_t v = 0;
        if (at + bytes > size) return 0;
        for (int i = bytes - 1; i >= 0; --i) v = (v << 8) | base[at + i];
        return v;
    };
    if (size >= 24 && std::string(code_object.data(), 24) == "__CLANG_OFFLOAD_BUNDLE__")
    {
        const uint64_t entries = rd(24, 8);
        size_t at = 32;
        for (uint64_t e = 0; e < entries; ++e)
        {
            const uint64_t offset = rd(at, 8), length = rd(at + 8, 8), triple = rd(at + 16, 8);
            at += 24 + triple;
            if (offset + length <= size && length >= 4 && std::string(code_object.data() + offset, 4) == "\x7f" "ELF")
            {
                base += offset;
                size = length;
                break;
            }
        }
    }
    if (size < 64 || std::string(reinterpret_cast<const char *>(base), 4) != "\x7f" "ELF" || base[4] != 2 || base[5] != 1) return -1;
    const uint64_t shoff = rd(0x28, 8), shentsize = rd(0x3A, 2), shnum = rd(0x3C, 2);
    const std::string wanted = function + ".kd";
    for (uint64_t i = 0; i < shnum; ++i)
    {
        const size_t sh = shoff + i * shentsize;
        const uint64_t type = rd(sh + 4, 4);
        if (type != 2 && type != 11) continue;  // SHT_SYMTAB, SHT_DYNSYM
        const uint64_t symoff = rd(sh + 0x18, 8), symsize = rd(sh + 0x20, 8), link = rd(sh + 0x28, 4), entsize = rd(sh + 0x38, 8);
        if (entsize == 0 || link >= shnum) continue;
        const size_t strsh = shoff + link * shentsize;
        const uint64_t stroff = rd(strsh + 0x18, 8), strsize = rd(strsh + 0x20, 8);
        for (uint64_t s = 0; s + entsize <= symsize; s += entsize)
        {
            const size_t sym = symoff + s;
            const uint64_t name = rd(sym, 4), shndx = rd(sym + 6, 2), value = rd(sym + 8, 8);
            if (name >= strsize || stroff + name + wanted.size() + 1 > size) continue;
            if (std::string(reinterpret_cast<const char *>(base) + stroff + name) != wanted) continue;
            if (shndx == 0 || shndx >= shnum) continue;
            const size_t sec = shoff + shndx * shentsize;
            const uint64_t addr = rd(sec + 0x10, 8), offset = rd(sec + 0x18, 8);
            const size_t descriptor = offset + (value - addr);
            if (descriptor + 64 > size) return -1;
            return static_cast<int>(rd(descriptor + 4, 4));
        }
    }
    return -1;
}

std::string HipKernel::FirstKernelWithPrivateMemory() const
{
    // Test hook: ACRO_HIP_TEST_PRIVATE_BYTES="first,second" stands for what the code object says on the first and on
    // the second (relief) compilation, so that both branches can be exercised with a kernel that does not spill.
    if (const char *env = std::getenv("ACRO_HIP_TEST_PRIVATE_BYTES"))
    {
        const std::string text(env);
        const size_t comma = text.find(',');
        const std::string mine = Relieved ? (comma == std::string::npos ? text : text.substr(comma + 1)) : text.substr(0, comma);
        return std::atoi(mine.c_str()) > 0 && !Guarded.empty() ? Guarded[0] : std::string();
    }
    for (const std::string &name : Guarded)
    {
        const int bytes = PrivateSegmentBytes(CodeObject, name);
        ACROBATIC_ASSERT(bytes >= 0, "Kernel " + name + " is not in the code object of " + FunctionName + ".");
        if (bytes > 0) return name;
    }
    return std::string();
}

HipKernel::HipKernel(const std::string &module_name, const std::string &source,
                     const std::vector<std::string> &no_private_memory, const std::string &relief_macro)
    : FunctionName(module_name), Source(source), CacheHit(false), Guarded(no_private_memory), Module(nullptr)
{
    // Experiment hook: $ACRO_HIP_KERNEL_OVERRIDE_DIR/<module name>.hip, when it exists, is compiled in place of the
    // generated source (same function names and parameters), e.g. a hand-edited copy of what GetImplementation printed.
    if (const char *dir = debugHooks() ? std::getenv("ACRO_HIP_KERNEL_OVERRIDE_DIR") : nullptr)
    {
        std::ifstream in(std::string(dir) + "/" + module_name + ".hip");
        if (in)
        {
            std::ostringstream text;
            text << in.rdbuf();
            Source = text.str();
            std::cerr << "acrotensor: " << module_name << " compiled from " << dir << "/" << module_name << ".hip" << std::endl;
        }
    }
    Compile();
    Spilling = FirstKernelWithPrivateMemory();
    if (!Spilling.empty() && !relief_macro.empty())
    {
        Source = "#define " + relief_macro + " 1\n" + Source;
        CacheHit = false;
        CodeObject.clear();
        Relieved = true;
        Compile();
        Spilling = FirstKernelWithPrivateMemory();
    }
}

HipKernel::~HipKernel()
{
    if (Module != nullptr) (void)hipModuleUnload(static_cast<hipModule_t>(Module));
}

void HipKernel::Compile()
{
    const std::string path = cachePath(FunctionName, Source);
    if (!path.empty())
    {
        std::ifstream in(path, std::ios::binary | std::ios::ate);
        if (in)
        {
            std::streamsize n = in.tellg();
            in.seekg(0);
            CodeObject.resize(static_cast<size_t>(n));
            if (n > 0 && in.read(CodeObject.data(), n))
            {
                CacheHit = true;
                return;
            }
            CodeObject.clear();
        }
    }

    hiprtcProgram prog;
    rtcCheck(hiprtcCreateProgram(&prog, Source.c_str(), (FunctionName + ".hip").c_str(), 0, nullptr, nullptr),
             "hiprtcCreateProgram");
    const std::vector<std::string> extra = extraCompileOptions();
    std::vector<const char *> options(kCompileOptions, kCompileOptions + kNumCompileOptions);
    for (const std::string &option : extra) options.push_back(option.c_str());
    hiprtcResult result = hiprtcCompileProgram(prog, static_cast<int>(options.size()), options.data());
    if (result != HIPRTC_SUCCESS)
    {
        size_t log_size = 0;
        hiprtcGetProgramLogSize(prog, &log_size);
        std::string log(log_size, '\0');
        if (log_size > 0) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        std::cerr << "---- generated kernel that failed to compile ----\n"
                  << Source << "\n---- compiler log ----\n"
                  << log << std::endl;
        throw_error("hipRTC compilation of " + FunctionName + " failed:\n" + log);
    }
    size_t code_size = 0;
    rtcCheck(hiprtcGetCodeSize(prog, &code_size), "hiprtcGetCodeSize");
    CodeObject.resize(code_size);
    rtcCheck(hiprtcGetCode(prog, CodeObject.data()), "hiprtcGetCode");
    hiprtcDestroyProgram(&prog);

    if (!path.empty() && makeDirs(cacheDir()))
    {
        // Write to a private name first so that a concurrent reader never sees a partial file.
        std::string tmp = path + ".tmp" + std::to_string(static_cast<long>(::getpid()));
        std::ofstream out(tmp, std::ios::binary);
        if (out && out.write(CodeObject.data(), static_cast<std::streamsize>(CodeObject.size())))
        {
            out.close();
            if (std::rename(tmp.c_str(), path.c_str()) != 0) std::remove(tmp.c_str());
        }
    }
}

void HipKernel::EnsureLoaded()
{
    if (Module != nullptr) return;
    // loading a code object allocates device memory for it
    ACROBATIC_ASSERT(!hip::NoAllocation::Active(),
                     "Kernel " + FunctionName + " is not loaded on the device yet, and a call that must not allocate "
                     "cannot load it: run the same operation once through the ordinary entry point before.");
    hipModule_t module;
    hipError_t err = hipModuleLoadData(&module, CodeObject.data());
    if (err != hipSuccess && CacheHit)
    {
        // A code object from the disk cache that does not load (damaged file, different driver): compile afresh.
        (void)hipGetLastError();
        const std::string path = cachePath(FunctionName, Source);
        if (!path.empty()) std::remove(path.c_str());
        CacheHit = false;
        CodeObject.clear();
        Compile();
        err = hipModuleLoadData(&module, CodeObject.data());
    }
    ACRO_HIP_CHECK(err);
    // What the compile-time check read from the kernel descriptors, confirmed by the loaded module.
    for (const std::string &name : Guarded)
    {
        hipFunction_t function;
        int privateBytes = 0;
        ACRO_HIP_CHECK(hipModuleGetFunction(&function, module, name.c_str()));
        ACRO_HIP_CHECK(hipFuncGetAttribute(&privateBytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, function));
        if (privateBytes > 0)
        {
            (void)hipModuleUnload(module);
            throw_error("Matrix-core kernel " + name + " was loaded with " + std::to_string(privateBytes) +
                        " bytes of private memory per work item (register spills): it is not launched.");
        }
    }
    Module = module;
}

void HipKernel::Launch(const std::string &function_name, unsigned grid, unsigned grid_y, unsigned block, void **args)
{
    ACROBATIC_ASSERT(Spilling.empty(), "Matrix-core kernel " + Spilling + " has private memory (register spills): it is not launched.");
    EnsureLoaded();
    auto it = Functions.find(function_name);
    if (it == Functions.end())
    {
        hipFunction_t function;
        ACRO_HIP_CHECK(hipModuleGetFunction(&function, static_cast<hipModule_t>(Module), function_name.c_str()));
        it = Functions.emplace(function_name, function).first;
    }
    ACRO_HIP_CHECK(hipModuleLaunchKernel(static_cast<hipFunction_t>(it->second), grid, grid_y, 1, block, 1, 1, 0,
                                         static_cast<hipStream_t>(hip::Stream()), args, nullptr));
}

void HipKernel::WriteCodeToFile(const std::string &path) const
{
    std::ofstream out(path);
    ACROBATIC_ASSERT(static_cast<bool>(out), "Can't open " + path + " for writing.");
    out << Source;
}

}  // namespace acro
