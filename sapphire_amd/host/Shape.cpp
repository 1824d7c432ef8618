#include <Sapphire/util/Shape.hpp>

#include <algorithm>
#include <numeric>
#include <stdexcept>

namespace Sapphire
{
std::size_t Shape::Resolve(int index, const char* who) const
{
    const int n = Dim();
    if (index >= n || index < -n)
        throw std::invalid_argument(std::string("Shape::") + who + " - Given index " +
                                    std::to_string(index) +
                                    " is out of range (Shape dimension : " + std::to_string(n) +
                                    ")");
    return static_cast<std::size_t>(index < 0 ? n + index : index);
}

int& Shape::operator[](int index)
{
    return m_dims[Resolve(index, "operator[]")];
}

int Shape::At(int index) const
{
    return m_dims[Resolve(index, "At")];
}

void Shape::Set(int index, int value)
{
    const std::size_t pos = Resolve(index, "Set");
    if (value == 0)
        throw std::invalid_argument("Shape::Set - Shape cannot have dimension with '0'");
    m_dims[pos] = value;
}

int Shape::Size() const noexcept
{
    if (m_dims.empty())
        return 0;
    return std::accumulate(m_dims.begin(), m_dims.end(), 1, [](int a, int b) { return a * b; });
}

std::string Shape::ToString() const
{
    std::string text = "Dim : " + std::to_string(Dim()) + "  [";
    for (int d : m_dims)
        text += std::to_string(d) + " ";
    return text + " ] ";
}

void Shape::Expand(int dim)
{
    if (dim < 0)
        throw std::invalid_argument("Shape::Expand - Given dimension " + std::to_string(dim) +
                                    " must be greater than zero");
    if (dim > Dim())
        m_dims.insert(m_dims.begin(), static_cast<std::size_t>(dim - Dim()), 1);
}

void Shape::Shrink(int dim)
{
    if (dim < 0)
        throw std::invalid_argument("Shape::Shrink - Given dimension " + std::to_string(dim) +
                                    " must be greater than zero");
    if (dim >= Dim())
        return;
    if (dim == 0)
        throw std::invalid_argument("Shape::Shrink - cannot shrink to zero dimensions");
    const auto cut = m_dims.begin() + (Dim() - dim);
    const int folded = std::accumulate(m_dims.begin(), cut, 1, [](int a, int b) { return a * b; });
    m_dims.erase(m_dims.begin(), cut);
    m_dims.front() *= folded;
}

void Shape::Squeeze(int index)
{
    const std::size_t fromFront = Resolve(index, "Squeeze");
    // the reference counts this position from the back
    const std::size_t pos = m_dims.size() - 1 - fromFront;
    if (m_dims[pos] == 1)
        m_dims.erase(m_dims.begin() + static_cast<std::ptrdiff_t>(pos));
}

void Shape::Squeeze()
{
    m_dims.erase(std::remove_if(m_dims.begin(), m_dims.end(), [](int d) { return d <= 1; }),
                 m_dims.end());
}

int Shape::GetNumUnits(int requiredDim) const
{
    if (requiredDim < 0)
        throw std::invalid_argument("Shape::GetNumUnits - Given dimension " +
                                    std::to_string(requiredDim) + " must be greater than zero");
    int units = 1;
    for (int i = 0; i < Dim() - requiredDim; ++i)
        units *= m_dims[static_cast<std::size_t>(i)];
    return units;
}

int Shape::GetUnitSize(int requiredDim) const
{
    if (requiredDim < 0)
        throw std::invalid_argument("Shape::GetUnitSize - Given dimension " +
                                    std::to_string(requiredDim) + " must be greater than zero");
    return Size() / GetNumUnits(requiredDim);
}

Shape Shape::GetTranspose() const
{
    if (m_dims.empty())
        throw std::runtime_error("GetTranspose - Shape cannot be empty  to perform transpose");
    std::vector<int> dims = m_dims;
    if (dims.size() == 1)
        dims.push_back(1);
    else
        std::swap(dims[dims.size() - 1], dims[dims.size() - 2]);
    return Shape(dims);
}
}  // namespace Sapphire
