#include <Sapphire/util/CudaDevice.hpp>

#include <sapphire_hip.h>

#include <cstdlib>
#include <cstring>
#include <stdexcept>

namespace Sapphire
{
int CudaDevice::GetAvailableCudaDeviceCount()
{
    int count = 0;
    sph_device_count(&count);
    return count;
}

CudaDevice::CudaDevice(int id, std::string name) : m_id(id), m_name(std::move(name))
{
    if (id >= GetAvailableCudaDeviceCount())
        throw std::runtime_error("Cuda device has not been detected");
    if (id >= 0)
    {
        SphDeviceInfo info;
        if (sph_device_info(id, &info) == SPH_OK && std::strncmp(info.arch, "gfx", 3) == 0)
            m_capability = std::atoi(info.arch + 3);
    }
}
}  // namespace Sapphire
