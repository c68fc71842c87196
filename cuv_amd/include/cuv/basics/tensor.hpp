// The subset of cuv::tensor the DIA path and its tests touch, without Boost.
//
// Mirrors src/cuv/basics/tensor.hpp of the reference for: the 1-d / 2-d /
// extents / shape-vector constructors (:688-741), the non-owning pointer
// views (:783-854), ptr() (:329-339), shape() (:317-319,389-393), size()
// (:360-367), ndim() (:310-312), operator()(i, j) (:502-515), operator[]
// (:439-477), same-type assignment that shares memory (:881-890), cross-space
// assignment that copies (:909-930) and dealloc() (:1121-1125).  Device
// elements are reached through a proxy that moves one value per access, like
// the reference's reference<T, dev_memory_space> (src/cuv/basics/reference.cu:18-28).
// N-d slicing, pitched memory and pooled allocators are not reproduced.
#ifndef __CUV_TENSOR_HPP__
#define __CUV_TENSOR_HPP__

#include <cstdlib>
#include <cstring>
#include <limits>
#include <memory>
#include <numeric>
#include <vector>

#include <cuv/basics/tags.hpp>
#include <cuv/tools/cuv_general.hpp>

namespace cuv {

// ---- extents[a][b] / indices[index_range(a, b)] -------------------------------
struct index_range {
    long start, finish;
    index_range() : start(0), finish(-1) {}
    index_range(long s, long f) : start(s), finish(f) {}
};

template <int D>
struct extent_gen {
    unsigned int ranges[D > 0 ? D : 1];
    extent_gen<D + 1> operator[](unsigned int n) const
    {
        extent_gen<D + 1> e;
        for (int i = 0; i < D; ++i) e.ranges[i] = ranges[i];
        e.ranges[D] = n;
        return e;
    }
};
template <int D>
struct index_gen {
    index_range ranges[D > 0 ? D : 1];
    index_gen<D + 1> operator[](const index_range &r) const
    {
        index_gen<D + 1> e;
        for (int i = 0; i < D; ++i) e.ranges[i] = ranges[i];
        e.ranges[D] = r;
        return e;
    }
};
static const extent_gen<0> extents = extent_gen<0>();
static const index_gen<0> indices = index_gen<0>();

// ---- raw storage ---------------------------------------------------------------
namespace detail {
template <class M> struct space;
template <> struct space<host_memory_space> {
    static void *alloc(size_t bytes)
    {
        void *p = std::malloc(bytes ? bytes : 1);
        if (!p) throw std::bad_alloc();
        return p;
    }
    static void free(void *p) { std::free(p); }
};
template <> struct space<dev_memory_space> {
    static void *alloc(size_t bytes)
    {
        void *p = nullptr;
        cuvSafeCall(hipMalloc(&p, bytes ? bytes : 1));
        return p;
    }
    static void free(void *p) { (void)hipFree(p); }
};
template <class MD, class MS> struct copy_kind;
template <> struct copy_kind<host_memory_space, host_memory_space> { static const hipMemcpyKind value = hipMemcpyHostToHost; };
template <> struct copy_kind<dev_memory_space, host_memory_space> { static const hipMemcpyKind value = hipMemcpyHostToDevice; };
template <> struct copy_kind<host_memory_space, dev_memory_space> { static const hipMemcpyKind value = hipMemcpyDeviceToHost; };
template <> struct copy_kind<dev_memory_space, dev_memory_space> { static const hipMemcpyKind value = hipMemcpyDeviceToDevice; };

template <class V, class MD, class MS>
inline void copy(V *dst, const V *src, size_t n)
{
    if (!n) return;
    if (copy_kind<MD, MS>::value == hipMemcpyHostToHost) std::memcpy(dst, src, n * sizeof(V));
    else cuvSafeCall(hipMemcpy(dst, src, n * sizeof(V), copy_kind<MD, MS>::value));
}
}  // namespace detail

template <class V, class M>
class memory {
    V *m_ptr;
    size_t m_size;
    memory(const memory &);
    memory &operator=(const memory &);
  public:
    explicit memory(size_t n) : m_ptr(static_cast<V *>(detail::space<M>::alloc(n * sizeof(V)))), m_size(n) {}
    ~memory() { detail::space<M>::free(m_ptr); }
    V *ptr() { return m_ptr; }
    size_t size() const { return m_size; }
};

// ---- element proxies -------------------------------------------------------------
template <class V, class M> struct reference;
template <class V> struct reference<V, host_memory_space> {
    V *p;
    explicit reference(V *q) : p(q) {}
    operator V() const { return *p; }
    reference &operator=(const V &v) { *p = v; return *this; }
    reference &operator=(const reference &o) { *p = (V)o; return *this; }
    reference &operator+=(const V &v) { *p += v; return *this; }
};
template <class V> struct reference<V, dev_memory_space> {
    V *p;
    explicit reference(V *q) : p(q) {}
    operator V() const
    {
        V v;
        cuvSafeCall(hipMemcpy(&v, p, sizeof(V), hipMemcpyDeviceToHost));
        return v;
    }
    reference &operator=(const V &v)
    {
        cuvSafeCall(hipMemcpy(p, &v, sizeof(V), hipMemcpyHostToDevice));
        return *this;
    }
    reference &operator=(const reference &o) { return *this = (V)o; }
};

// ---- tensor ------------------------------------------------------------------------
template <class V, class M, class L = row_major>
class tensor {
  public:
    typedef V value_type;
    typedef M memory_space_type;
    typedef L memory_layout_type;
    typedef unsigned int size_type;
    typedef int index_type;
    typedef reference<V, M> reference_type;
    typedef memory<V, M> memory_type;

  private:
    std::vector<size_type> m_shape;
    std::shared_ptr<memory_type> m_memory;   // empty for views
    V *m_ptr;

    static void check_size_limit(size_t n)
    {
        if (n > static_cast<size_t>(std::numeric_limits<index_type>::max()))
            throw std::runtime_error("maximum tensor size exceeded");
    }
    void allocate()
    {
        size_t n = 1;
        for (size_t i = 0; i < m_shape.size(); ++i) n *= m_shape[i];
        check_size_limit(n);
        m_memory.reset(new memory_type(n));
        m_ptr = m_memory->ptr();
    }
    size_t linear(size_type i, size_type j) const
    {
        // column_major: first index runs fastest
        return std::is_same<L, column_major>::value ? (size_t)j * m_shape[0] + i : (size_t)i * m_shape[1] + j;
    }

  public:
    tensor() : m_ptr(nullptr) {}
    explicit tensor(size_type n) : m_shape(1, n), m_ptr(nullptr) { allocate(); }
    explicit tensor(int n) : m_shape(1, (size_type)n), m_ptr(nullptr) { cuvAssert(n >= 0); allocate(); }
    tensor(size_type h, size_type w) : m_ptr(nullptr) { m_shape.push_back(h); m_shape.push_back(w); allocate(); }
    tensor(int h, int w) : m_ptr(nullptr) { m_shape.push_back((size_type)h); m_shape.push_back((size_type)w); allocate(); }
    template <int D>
    explicit tensor(const extent_gen<D> &e) : m_shape(e.ranges, e.ranges + D), m_ptr(nullptr) { allocate(); }
    explicit tensor(const std::vector<size_type> &shape) : m_shape(shape), m_ptr(nullptr) { allocate(); }

    // views over memory the caller owns
    template <int D>
    tensor(const extent_gen<D> &e, V *ptr) : m_shape(e.ranges, e.ranges + D), m_ptr(ptr) {}
    template <int D>
    tensor(const index_gen<D> &idx, V *ptr) : m_ptr(ptr)
    {
        for (int i = 0; i < D; ++i) m_shape.push_back((size_type)(idx.ranges[i].finish - idx.ranges[i].start));
    }

    // same type: O(1), shares the memory
    tensor(const tensor &o) : m_shape(o.m_shape), m_memory(o.m_memory), m_ptr(o.m_ptr) {}
    tensor &operator=(const tensor &o)
    {
        m_shape = o.m_shape; m_memory = o.m_memory; m_ptr = o.m_ptr;
        return *this;
    }
    // other memory space: allocates if the size differs, then copies
    template <class OM>
    explicit tensor(const tensor<V, OM, L> &o) : m_ptr(nullptr) { *this = o; }
    template <class OM>
    tensor &operator=(const tensor<V, OM, L> &o)
    {
        if (!m_ptr || size() != o.size()) { m_shape = o.shape(); allocate(); }
        else m_shape = o.shape();
        detail::copy<V, M, OM>(m_ptr, o.ptr(), size());
        return *this;
    }

    index_type ndim() const { return (index_type)m_shape.size(); }
    std::vector<size_type> shape() const { return m_shape; }
    size_type shape(size_t i) const { return m_shape[i]; }
    size_type size() const
    {
        if (m_shape.empty()) return 0;
        size_t n = 1;
        for (size_t i = 0; i < m_shape.size(); ++i) n *= m_shape[i];
        return (size_type)n;
    }
    size_type memsize() const { return size() * sizeof(V); }
    V *ptr() { return m_ptr; }
    const V *ptr() const { return m_ptr; }
    void dealloc() { m_memory.reset(); m_ptr = nullptr; m_shape.clear(); }
    void reshape(size_type h, size_type w)
    {
        cuvAssert((size_t)h * w == size());
        m_shape.clear(); m_shape.push_back(h); m_shape.push_back(w);
    }

    reference_type operator[](index_type i) { return reference_type(m_ptr + i); }
    const reference_type operator[](index_type i) const { return reference_type(const_cast<V *>(m_ptr) + i); }
    reference_type operator()(index_type i, index_type j) { return reference_type(m_ptr + linear(i, j)); }
    const reference_type operator()(index_type i, index_type j) const { return reference_type(const_cast<V *>(m_ptr) + linear(i, j)); }
};

}  // namespace cuv
#endif
