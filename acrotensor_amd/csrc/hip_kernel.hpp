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
    HipKernel(const std::string &module_name, const std::string &source);
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

  private:
    void Compile();
    void EnsureLoaded();

    std::string FunctionName;
    std::string Source;
    std::vector<char> CodeObject;
    bool CacheHit;
    void *Module;                            // hipModule_t
    std::map<std::string, void *> Functions;  // hipFunction_t by name
};

}  // namespace acro

#endif
