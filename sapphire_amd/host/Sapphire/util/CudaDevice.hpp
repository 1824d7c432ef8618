// Device descriptor and execution-mode switch of the operator layer.
//
// The names CudaDevice and ComputeMode::Cuda are the reference's
// (Includes/Sapphire/util/CudaDevice.hpp:16-60) and are kept so that code written
// against it compiles unchanged; here they denote a HIP device (MI355X, gfx950).
#ifndef SAPPHIRE_AMD_UTIL_CUDADEVICE_HPP
#define SAPPHIRE_AMD_UTIL_CUDADEVICE_HPP

#include <string>

namespace Sapphire
{
enum class ComputeMode
{
    Host,
    Cuda,
};

class CudaDevice
{
public:
    //! An unconfigured descriptor (id -1): tensors built with it live on the host only.
    CudaDevice() = default;
    //! Throws std::runtime_error("Cuda device has not been detected") when `id` is not below
    //! the number of visible devices (Sources/Sapphire/util/CudaDevice.cpp:16-19).
    CudaDevice(int id, std::string name);

    bool operator==(const CudaDevice& other) const { return m_id == other.m_id && m_name == other.m_name; }
    bool operator!=(const CudaDevice& other) const { return !(*this == other); }

    [[nodiscard]] std::string Name() const { return m_name; }
    [[nodiscard]] int GetID() const { return m_id; }
    //! The reference reports major*10+minor of the CUDA capability; here the number of
    //! the gfx target (950 on MI355X), 0 when unconfigured.
    [[nodiscard]] int GetCudaCapability() const { return m_capability; }

    static int GetAvailableCudaDeviceCount();

private:
    int m_id = -1;
    std::string m_name = "Undefined";
    int m_capability = 0;
};
}  // namespace Sapphire

#endif
