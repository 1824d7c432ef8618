// Shape of a tensor: an ordered list of positive extents, last one fastest.
//
// Same interface and results as the reference's Sapphire::Shape
// (Includes/Sapphire/util/Shape.hpp:22-95, Sources/Sapphire/util/shape.cpp), which the
// operator layer uses to derive M, N, K and to walk the batch dimensions.
#ifndef SAPPHIRE_AMD_UTIL_SHAPE_HPP
#define SAPPHIRE_AMD_UTIL_SHAPE_HPP

#include <initializer_list>
#include <string>
#include <vector>

namespace Sapphire
{
enum class Type
{
    Sparse,
    Dense,
};

class Shape
{
public:
    Shape() = default;
    Shape(std::initializer_list<int> dims) : m_dims(dims) {}
    explicit Shape(std::vector<int> dims) : m_dims(std::move(dims)) {}

    bool operator==(const Shape& other) const { return m_dims == other.m_dims; }
    bool operator!=(const Shape& other) const { return m_dims != other.m_dims; }

    //! Extent at `index`; negative indices count from the end.  Throws
    //! std::invalid_argument when out of range.
    int& operator[](int index);
    [[nodiscard]] int At(int index) const;
    void Set(int index, int value);

    [[nodiscard]] int Dim() const { return static_cast<int>(m_dims.size()); }
    //! Product of the extents in int arithmetic; 0 for an empty shape.
    [[nodiscard]] int Size() const noexcept;
    [[nodiscard]] std::vector<int> GetShapeVector() const { return m_dims; }
    [[nodiscard]] std::string ToString() const;

    //! Second-to-last extent, 1 when there are fewer than two.
    [[nodiscard]] int Rows() const { return m_dims.size() > 1 ? m_dims[m_dims.size() - 2] : 1; }
    //! Last extent, 0 when empty.
    [[nodiscard]] int Cols() const { return m_dims.empty() ? 0 : m_dims.back(); }

    //! Pads with leading 1s up to `dim` extents; no effect when already that long.
    void Expand(int dim);
    //! Keeps the trailing `dim` extents and folds every dropped leading one into the first kept.
    void Shrink(int dim);
    //! Drops the extent `index` positions from the end when it is 1.
    void Squeeze(int index);
    //! Drops every extent equal to 1.
    void Squeeze();

    //! Product of the leading Dim() - requiredDim extents (1 when there are none).
    [[nodiscard]] int GetNumUnits(int requiredDim) const;
    [[nodiscard]] int GetUnitSize(int requiredDim) const;
    //! Last two extents swapped; a 1-D shape [n] becomes [n, 1].
    [[nodiscard]] Shape GetTranspose() const;

private:
    [[nodiscard]] std::size_t Resolve(int index, const char* who) const;

    std::vector<int> m_dims;
};
}  // namespace Sapphire

#endif
