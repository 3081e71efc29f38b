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

// Experiment hook: further options for the run-time compiler, separated by blanks (ACRO_HIP_COMPILE_OPTIONS="-mllvm
// -amdgpu-..."); they are part of the key of the on-disk cache.
std::vector<std::string> extraCompileOptions()
{
    std::vector<std::string> extra;
    const char *env = std::getenv("ACRO_HIP_COMPILE_OPTIONS");
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

HipKernel::HipKernel(const std::string &module_name, const std::string &source)
    : FunctionName(module_name), Source(source), CacheHit(false), Module(nullptr)
{
    // Experiment hook: $ACRO_HIP_KERNEL_OVERRIDE_DIR/<module name>.hip, when it exists, is compiled in place of the
    // generated source (same function names and parameters), e.g. a hand-edited copy of what GetImplementation printed.
    if (const char *dir = std::getenv("ACRO_HIP_KERNEL_OVERRIDE_DIR"))
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
    // Kernels that keep no arrays in private memory by design (the matrix-core schedules) carry a switch that trades
    // registers for LDS reads.  When the compiler has fit one of them into the registers only with spills, compile
    // the module again with the switch on: spill code around the matrix-core accumulators is slow, and the compiler
    // has been seen to lose half of a spilled 64-bit value there (a result off in its low 32 bits).
    static const char *const kSwitch = "ACRO_KEEP_OPERATOR_IN_LDS";
    if (Source.find(std::string("#ifdef ") + kSwitch) != std::string::npos && Source.compare(0, 8, "#define ") != 0)
    {
        bool spills = false;
        for (size_t at = Source.find("__global__"); at != std::string::npos && !spills; at = Source.find("__global__", at + 1))
        {
            const size_t name = Source.find("void ", at), paren = Source.find('(', name);
            if (name == std::string::npos || paren == std::string::npos) break;
            hipFunction_t function;
            int privateBytes = 0;
            ACRO_HIP_CHECK(hipModuleGetFunction(&function, module, Source.substr(name + 5, paren - name - 5).c_str()));
            ACRO_HIP_CHECK(hipFuncGetAttribute(&privateBytes, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, function));
            spills = privateBytes > 0;
        }
        if (spills)
        {
            ACRO_HIP_CHECK(hipModuleUnload(module));
            Source = std::string("#define ") + kSwitch + " 1\n" + Source;
            CacheHit = false;
            CodeObject.clear();
            Compile();
            ACRO_HIP_CHECK(hipModuleLoadData(&module, CodeObject.data()));
        }
    }
    Module = module;
}

void HipKernel::Launch(const std::string &function_name, unsigned grid, unsigned grid_y, unsigned block, void **args)
{
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
