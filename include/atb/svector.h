// atb::SVector<T> - the small fixed-capacity vector that carries tensors and
// tensor descriptions across the ATB operator API.
//
// Same public surface, limits and object layout as the reference container
// (reference include/atb/svector.h:27-110 for the limits and constructors,
// :585-589 for the member order), so a VariantPack filled by existing caller
// code means the same thing here:
//   * up to DEFAULT_SVECTOR_SIZE (64) elements live inside the object,
//   * past that the elements move to one malloc'ed block of MAX_SVECTOR_SIZE,
//   * anything beyond 256 throws MaxSizeExceeded.
#ifndef ATB_SVECTOR_H
#define ATB_SVECTOR_H
#include <cstddef>
#include <cstdlib>
#include <exception>
#include <initializer_list>
#include <new>
#include <ostream>
#include <stdexcept>
#include <type_traits>

namespace atb {
constexpr std::size_t MAX_SVECTOR_SIZE = 256;
constexpr std::size_t DEFAULT_SVECTOR_SIZE = 64;
constexpr bool CHECK_BOUND = true;

struct MaxSizeExceeded : public std::exception {};

template <class T> class SVector {
public:
    constexpr SVector() : size_(0)
    {
        for (std::size_t i = 0; i < DEFAULT_SVECTOR_SIZE; ++i) {
            storage_[i] = {};
        }
    }

    SVector(std::initializer_list<T> list)
    {
        if (list.size() > MAX_SVECTOR_SIZE) {
            throw MaxSizeExceeded();
        }
        if (list.size() > DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, 0);
        }
        T *dst = Base();
        for (const T &v : list) {
            dst[size_++] = v;
        }
    }

    explicit SVector(std::size_t size, const T &value = 0)
    {
        if (size > MAX_SVECTOR_SIZE) {
            throw MaxSizeExceeded();
        }
        if (size > DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, 0);
        }
        T *dst = Base();
        for (std::size_t i = 0; i < size; ++i) {
            dst[i] = value;
        }
        size_ = size;
    }

    SVector(const SVector<T> &other)
    {
        CopyFrom(other);
    }

    ~SVector()
    {
        if (heap_) {
            free(heap_);
        }
    }

    SVector &operator=(const SVector &other)
    {
        if (this != &other) {
            Release();
            CopyFrom(other);
        }
        return *this;
    }

    SVector &operator=(std::initializer_list<T> list)
    {
        if (list.size() > MAX_SVECTOR_SIZE) {
            throw MaxSizeExceeded();
        }
        Release();
        if (list.size() > DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, 0);
        }
        T *dst = Base();
        for (const T &v : list) {
            dst[size_++] = v;
        }
        return *this;
    }

    void push_back(const T &val) noexcept((!CHECK_BOUND) && std::is_nothrow_assignable<T, const T &>::value)
    {
        if (!heap_ && size_ == DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, size_);
        }
        if (heap_ && CHECK_BOUND && size_ == capacity_) {
            throw MaxSizeExceeded();
        }
        Base()[size_++] = val;
    }

    void insert(const std::size_t pos, const T &value)
    {
        if (pos > size_) {
            throw std::out_of_range("SVector insert index out of stack range");
        }
        if (!heap_ && size_ == DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, size_);
        }
        if (heap_ && size_ == capacity_) {
            throw MaxSizeExceeded();
        }
        T *p = Base();
        for (std::size_t i = size_; i != pos; --i) {
            p[i] = p[i - 1];
        }
        p[pos] = value;
        ++size_;
    }

    T *begin() noexcept { return Base(); }
    const T *begin() const noexcept { return Base(); }
    T *end() noexcept { return Base() + size_; }
    const T *end() const noexcept { return Base() + size_; }
    T *data() noexcept { return Base(); }
    const T *data() const noexcept { return Base(); }

    T &operator[](std::size_t i)
    {
        BoundCheck(i, "SVector operator[] index out of range");
        return Base()[i];
    }
    const T &operator[](std::size_t i) const
    {
        BoundCheck(i, "SVector operator[] index out of range");
        return Base()[i];
    }
    T &at(std::size_t i)
    {
        BoundCheck(i, "SVector at index out of range");
        return Base()[i];
    }
    const T &at(std::size_t i) const
    {
        BoundCheck(i, "SVector at index out of range");
        return Base()[i];
    }

    std::size_t size() const noexcept { return size_; }
    bool empty() const noexcept { return size_ == 0; }
    void clear() noexcept { size_ = 0; }

    // Sets the element count; grows into the heap block when it passes the
    // inline capacity. New elements keep whatever the storage held.
    void resize(std::size_t size)
    {
        if (size > MAX_SVECTOR_SIZE || (heap_ && size > capacity_)) {
            throw MaxSizeExceeded();
        }
        if (!heap_ && size > DEFAULT_SVECTOR_SIZE) {
            Spill(MAX_SVECTOR_SIZE, size_);
        }
        size_ = size;
    }

    // Pre-allocates a heap block of exactly `size` default-initialised
    // elements when `size` does not fit inline; a no-op otherwise.
    void reserve(std::size_t size)
    {
        if (size > MAX_SVECTOR_SIZE) {
            throw MaxSizeExceeded();
        }
        if (size > DEFAULT_SVECTOR_SIZE) {
            if (heap_) {
                free(heap_);
                heap_ = nullptr;
            }
            Spill(size, 0);
            for (std::size_t i = 0; i < size; ++i) {
                heap_[i] = {};
            }
        }
    }

    bool operator==(const SVector<T> &other) const
    {
        if (size_ != other.size_) {
            return false;
        }
        const T *a = Base();
        const T *b = other.Base();
        for (std::size_t i = 0; i < size_; ++i) {
            if (!(a[i] == b[i])) {
                return false;
            }
        }
        return true;
    }
    bool operator!=(const SVector<T> &other) const { return !(*this == other); }

    // Shorter sorts first; equal lengths compare element by element.
    bool operator<(const SVector<T> &other) const
    {
        if (size_ != other.size_) {
            return size_ < other.size_;
        }
        const T *a = Base();
        const T *b = other.Base();
        for (std::size_t i = 0; i < size_; ++i) {
            if (a[i] < b[i]) {
                return true;
            }
            if (b[i] < a[i]) {
                return false;
            }
        }
        return false;
    }

private:
    // Member order and types mirror the reference object layout.
    std::size_t capacity_ = 0;
    std::size_t size_ = 0;
    T storage_[DEFAULT_SVECTOR_SIZE + 1];
    T *heap_ = nullptr;

    T *Base() noexcept { return heap_ ? heap_ : storage_; }
    const T *Base() const noexcept { return heap_ ? heap_ : storage_; }

    void BoundCheck(std::size_t i, const char *what) const
    {
        if (CHECK_BOUND && (i >= size_ || (!heap_ && i >= DEFAULT_SVECTOR_SIZE))) {
            throw std::out_of_range(what);
        }
    }

    // Allocates the heap block and carries over the first `keep` inline items.
    void Spill(std::size_t capacity, std::size_t keep)
    {
        T *block = reinterpret_cast<T *>(malloc(capacity * sizeof(T)));
        if (!block) {
            throw std::bad_alloc();
        }
        for (std::size_t i = 0; i < keep && i < DEFAULT_SVECTOR_SIZE; ++i) {
            block[i] = storage_[i];
        }
        heap_ = block;
        capacity_ = capacity;
    }

    void Release() noexcept
    {
        if (heap_) {
            free(heap_);
            heap_ = nullptr;
        }
        capacity_ = 0;
        size_ = 0;
    }

    void CopyFrom(const SVector<T> &other)
    {
        if (other.heap_) {
            Spill(other.capacity_ ? other.capacity_ : MAX_SVECTOR_SIZE, 0);
        }
        T *dst = Base();
        const T *src = other.Base();
        for (std::size_t i = 0; i < other.size_; ++i) {
            dst[i] = src[i];
        }
        size_ = other.size_;
    }
};

template <class T> std::ostream &operator<<(std::ostream &os, const SVector<T> &v)
{
    for (std::size_t i = 0; i < v.size(); ++i) {
        if (i) {
            os << ",";
        }
        os << v.at(i);
    }
    return os;
}
} // namespace atb
#endif
