// Front-end stand-in for <absl/types/span.h>: see ../../README.md.
#pragma once
#include <cstddef>
#include <type_traits>
#include <vector>
namespace absl {
template <typename T>
class Span {
public:
    using value_type = std::remove_cv_t<T>;
    using pointer = T*;
    using const_pointer = const T*;
    using reference = T&;
    using const_reference = const T&;
    using iterator = T*;
    using const_iterator = const T*;
    using size_type = std::size_t;
    constexpr Span() noexcept = default;
    constexpr Span(T* data, std::size_t size) noexcept : data_{data}, size_{size} {}
    template <std::size_t N>
    constexpr Span(T (&a)[N]) noexcept : data_{a}, size_{N} {}  // NOLINT
    template <typename V, typename = decltype(std::declval<V&>().data()), typename = decltype(std::declval<V&>().size())>
    constexpr Span(V& v) noexcept : data_{v.data()}, size_{v.size()} {}  // NOLINT
    template <typename V, typename = decltype(std::declval<const V&>().data()), typename = decltype(std::declval<const V&>().size()),
              typename = std::enable_if_t<std::is_const<T>::value, V>>
    constexpr Span(const V& v) noexcept : data_{v.data()}, size_{v.size()} {}  // NOLINT
    constexpr T* data() const noexcept { return data_; }
    constexpr std::size_t size() const noexcept { return size_; }
    constexpr bool empty() const noexcept { return size_ == 0; }
    constexpr T& operator[](std::size_t i) const noexcept { return data_[i]; }
    constexpr T* begin() const noexcept { return data_; }
    constexpr T* end() const noexcept { return data_ + size_; }
    constexpr T& front() const noexcept { return data_[0]; }
    constexpr T& back() const noexcept { return data_[size_ - 1]; }

private:
    T* data_ = nullptr;
    std::size_t size_ = 0;
};
template <typename T>
constexpr Span<T> MakeSpan(T* p, std::size_t n) noexcept { return Span<T>(p, n); }
template <typename T>
constexpr Span<T> MakeSpan(T* first, T* last) noexcept { return Span<T>(first, static_cast<std::size_t>(last - first)); }
template <typename C>
constexpr auto MakeSpan(C& c) noexcept { return Span<std::remove_pointer_t<decltype(c.data())>>(c.data(), c.size()); }
template <typename T>
constexpr Span<const T> MakeConstSpan(const T* p, std::size_t n) noexcept { return Span<const T>(p, n); }
template <typename T>
constexpr Span<const T> MakeConstSpan(const T* first, const T* last) noexcept { return Span<const T>(first, static_cast<std::size_t>(last - first)); }
template <typename C>
constexpr auto MakeConstSpan(const C& c) noexcept { return Span<const std::remove_pointer_t<decltype(c.data())>>(c.data(), c.size()); }
}  // namespace absl
