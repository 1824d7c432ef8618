// Plain stochastic gradient descent on TensorData, z <- z - learningRate * dz
// (Includes/Sapphire/operations/optimizers/SGD.hpp, Sources/Sapphire/operations/optimizers/SGD.cpp:22-28).
//
// The reference scales dz into a temporary and subtracts it (two passes, five array
// transfers).  Fused mode does both in one pass over z and dz; the product is still rounded
// to fp32 before the subtraction, so both modes give the same bits.
#ifndef SAPPHIRE_AMD_OPERATIONS_OPTIMIZERS_SGD_HPP
#define SAPPHIRE_AMD_OPERATIONS_OPTIMIZERS_SGD_HPP

#include <Sapphire/tensor/TensorData.hpp>

#include <string>

namespace Sapphire::Optimizer
{
class SGD
{
public:
    explicit SGD(float learningRate, bool fused = true)
        : m_learningRate(learningRate), m_fused(fused)
    {
    }

    //! Updates z in place.  z and dz must be in the same (device) mode.
    void operator()(TensorUtil::TensorData& z, const TensorUtil::TensorData& dz,
                    const std::string& name = std::string()) const;

    [[nodiscard]] float LearningRate() const { return m_learningRate; }
    //! One-pass device forms of the update may stand in for Scale + Sub (same result bits).
    [[nodiscard]] bool Fused() const { return m_fused; }

private:
    float m_learningRate;
    bool m_fused;
};
}  // namespace Sapphire::Optimizer

#endif
