// Runtime compiler and launcher for generated kernels: HIP C++ source -> hipRTC -> gfx950 code object ->
// hipModule -> hipModuleLaunchKernel on the library's stream.  Takes the place of the reference's CudaKernel
// (util/CudaUtil.hpp:29-57, util/CudaUtil.cpp:43-119: NVRTC -> PTX -> cuModule -> cuLaunchKernel).
//
// Compilation needs no device, so sources can be generated, compiled and inspected on a machine without a GPU;
// the code object is loaded into the device on the first launch.  Code objects are cached on disk keyed by a
// hash of source and options (directory $ACRO_HIP_CACHE_DIR, default $HOME/.cache/acrotensor_hip; set
// ACRO_HIP_CACHE_DIR=off to disable).
#ifndef ACRO_HIP_KERNEL_HPP
#define ACRO_HIP_KERNEL_HPP

#include <map>
#include <string>
#include <vector>

namespace acro
{

class HipKernel
{
  public:
    // Compiles immediately; throws std::runtime_error carrying the compiler log on failure.  module_name labels
    // the translation unit; the source may define several extern "C" __global__ functions.
    //
    // no_private_memory names kernels that must come out of the compiler without private memory (matrix-core
    // kernels: spill code around their accumulators has been seen to lose half of a 64-bit value).  Their private
    // segment size is read from the kernel descriptors of the code object, so the check needs no device.  When one
    // of them has private memory and relief_macro is not empty, the source is compiled once more with that macro
    // defined and checked again; what is left then is reported by PrivateMemoryRemains() and Launch refuses to run
    // such a module (the caller generates another schedule).
    HipKernel(const std::string &module_name, const std::string &source,
              const std::vector<std::string> &no_private_memory = std::vector<std::string>(),
              const std::string &relief_macro = std::string());
    ~HipKernel();
    HipKernel(const HipKernel &) = delete;
    HipKernel &operator=(const HipKernel &) = delete;

    // args: one pointer per kernel parameter (as for hipModuleLaunchKernel)
    void Launch(const std::string &function_name, unsigned grid, unsigned grid_y, unsigned block, void **args);

    const std::string &GetSource() const { return Source; }
    const std::string &GetModuleName() const { return FunctionName; }
    void WriteCodeToFile(const std::string &path) const;
    size_t GetCodeObjectSize() const { return CodeObject.size(); }
    bool WasCacheHit() const { return CacheHit; }
    // Name of a guarded kernel that still has private memory ("" when none has), and whether the relief macro was needed.
    const std::string &PrivateMemoryRemains() const { return Spilling; }
    bool ReliefApplied() const { return Relieved; }
    // Bytes of private memory per work item that the code object declares for `function` (its kernel descriptor's
    // private_segment_fixed_size); -1 when the code object holds no such kernel.
    static int PrivateSegmentBytes(const std::vector<char> &code_object, const std::string &function);
    int PrivateSegmentBytes(const std::string &function) const { return PrivateSegmentBytes(CodeObject, function); }

  private:
    void Compile();
    void EnsureLoaded();
    std::string FirstKernelWithPrivateMemory() const;

    std::string FunctionName;
    std::string Source;
    std::vector<char> CodeObject;
    bool CacheHit;
    std::vector<std::string> Guarded;  // kernels that must not have private memory
    std::string Spilling;              // one of them that has it all the same (after the relief macro, if any)
    bool Relieved = false;
    void *Module;                            // hipModule_t
    std::map<std::string, void *> Functions;  // hipFunction_t by name
};

}  // namespace acro

#endif
