// DIA (diagonal) sparse matrix container.
//
// Mirrors src/cuv/basics/dia_matrix.hpp:57-276 of the reference: an offset
// table in table order, one value vector of stride*num_dia entries in which
// element (i, j) sits at vec[d*stride + i] with offsets[d] == j - i/row_fact,
// a map from offset to table position, and an assignment operator that takes
// the value vector away from its source.
//
// Two additions the MI355X path needs, both invisible to reference-style code:
//   * a host copy of the offset table (on the device the table lives in
//     device memory and every element read is a copy), refreshed by
//     set_offsets() / post_update_offsets();
//   * for dev_memory_space, a lazily built cuvdia descriptor (the run table
//     the kernels walk), dropped whenever the offsets change.
// The implicit shallow copy constructor of the reference (which would free the
// value vector twice) is deleted.
#ifndef __CUV_DIA_MATRIX_HPP__
#define __CUV_DIA_MATRIX_HPP__

#include <algorithm>
#include <iostream>
#include <map>
#include <memory>
#include <vector>

#include <cuv/basics/matrix.hpp>
#include <cuv/basics/tensor.hpp>
#include <cuv/tensor_ops/tensor_ops.hpp>
#include <cuv/tools/cuv_general.hpp>

namespace cuv {

template <class __value_type, class __memory_space_type, class __index_type = unsigned int>
class dia_matrix : public matrix<__value_type, __index_type> {
  public:
    typedef __value_type value_type;
    typedef const value_type const_value_type;
    typedef matrix<__value_type, __index_type> base_type;
    typedef __memory_space_type memory_space_type;
    typedef typename base_type::index_type index_type;
    typedef const tensor<value_type, memory_space_type> const_vec_type;
    typedef tensor<value_type, memory_space_type> vec_type;
    typedef tensor<int, memory_space_type> intvec_type;
    typedef dia_matrix<value_type, memory_space_type, index_type> my_type;
    typedef value_type *ptr_type;

  public:
    int m_num_dia;                       ///< number of diagonals stored
    unsigned int m_stride;               ///< how long the stored diagonals are
    vec_type *m_vec;                     ///< stores the actual data
    intvec_type m_offsets;               ///< stores the offsets of the diagonals
    std::map<int, index_type> m_dia2off; ///< maps a diagonal to a table position
    int m_row_fact;                      ///< steepness of the diagonals

  private:
    std::vector<int> m_offsets_host;                 // host copy of m_offsets, table order
    mutable std::shared_ptr<cuvdia_desc> m_desc;     // dev_memory_space only

    dia_matrix(const dia_matrix &);                  // not copyable (see header comment)

  public:
    ~dia_matrix() { dealloc(); }

    dia_matrix() : base_type(0, 0), m_num_dia(0), m_stride(0), m_vec(0), m_row_fact(0) {}

    dia_matrix(const index_type &h, const index_type &w, const int &num_dia, const int &stride, int row_fact = 1)
        : base_type(h, w), m_num_dia(num_dia), m_stride(stride), m_vec(NULL), m_offsets(num_dia),
          m_offsets_host(num_dia, 0)
    {
        m_row_fact = row_fact;
        cuvAssert(m_row_fact > 0);
        alloc();
    }
    void dealloc()
    {
        if (m_vec) delete m_vec;
        m_vec = NULL;
    }
    std::vector<index_type> shape() const
    {
        std::vector<index_type> s(2);
        s[0] = this->h();
        s[1] = this->w();
        return s;
    }
    void alloc()
    {
        cuvAssert(m_stride >= this->h() || m_stride >= this->w());
        m_vec = new vec_type((unsigned int)(m_stride * m_num_dia));
    }
    inline const vec_type &vec() const { return *m_vec; }
    inline vec_type &vec() { return *m_vec; }
    inline const vec_type *vec_ptr() const { return m_vec; }
    inline vec_type *vec_ptr() { return m_vec; }
    inline ptr_type ptr() { return m_vec->ptr(); }
    inline ptr_type ptr() const { return m_vec->ptr(); }
    inline int num_dia() const { return m_num_dia; }
    inline unsigned int stride() const { return m_stride; }
    inline int row_fact() const { return m_row_fact; }

    // ---- offsets ------------------------------------------------------------
    template <class T>
    void set_offsets(T begin, const T &end)
    {
        std::vector<int> v;
        while (begin != end) v.push_back((int)*begin++);
        store_offsets(v);
    }
    template <class T>
    void set_offsets(const std::vector<T> &v)
    {
        std::vector<int> w(v.begin(), v.end());
        store_offsets(w);
    }
    /// Re-reads the offset tensor (call after writing get_offsets() by hand).
    void post_update_offsets()
    {
        m_offsets_host.resize(m_offsets.size());
        detail::copy<int, host_memory_space, memory_space_type>(m_offsets_host.data(), m_offsets.ptr(),
                                                                m_offsets_host.size());
        rebuild_map();
    }
    inline void set_offset(const index_type &idx, const index_type &val)
    {
        m_offsets[idx] = (int)val;
        m_offsets_host[idx] = (int)val;
        m_dia2off[(int)val] = idx;
        m_desc.reset();
    }
    inline const_vec_type *get_dia(const int &k) const
    {
        typename std::map<int, index_type>::const_iterator it = m_dia2off.find(k);
        cuvAssert(it != m_dia2off.end());
        return new const_vec_type(indices[index_range(0, m_stride)], m_vec->ptr() + it->second * m_stride);
    }
    inline vec_type *get_dia(const int &k)
    {
        typename std::map<int, index_type>::const_iterator it = m_dia2off.find(k);
        cuvAssert(it != m_dia2off.end());
        return new vec_type(indices[index_range(0, m_stride)], m_vec->ptr() + it->second * m_stride);
    }
    inline const intvec_type &get_offsets() const { return m_offsets; }
    inline intvec_type &get_offsets() { return m_offsets; }
    inline int get_offset(const index_type &idx) const { return m_offsets_host[idx]; }
    /// Host copy of the offset table, in table order.
    inline const std::vector<int> &host_offsets() const { return m_offsets_host; }

    // ---- element access -----------------------------------------------------
    void set(const index_type &i, const index_type &j, const value_type &val)
    {
        int off = (int)j - (int)i / m_row_fact;
        typename std::map<int, index_type>::const_iterator it = m_dia2off.find(off);
        if (it == m_dia2off.end()) return;
        (*m_vec)[it->second * m_stride + i] = val;
    }
    value_type operator()(const index_type &i, const index_type &j) const
    {
        int off = (int)j - (int)i / m_row_fact;
        typename std::map<int, index_type>::const_iterator it = m_dia2off.find(off);
        if (it == m_dia2off.end()) return (value_type)0;
        return (*m_vec)[it->second * m_stride + i];
    }
    bool has(const index_type &i, const index_type &j) const
    {
        int off = (int)j - (int)i / m_row_fact;
        return m_dia2off.find(off) != m_dia2off.end();
    }

    /// Takes the value vector of `o` (which is left without one), like the reference.
    my_type &operator=(const my_type &o)
    {
        if (this == &o) return *this;
        this->dealloc();
        (base_type &)(*this) = (base_type &)o;
        m_vec = o.m_vec;
        m_num_dia = o.m_num_dia;
        m_stride = o.m_stride;
        m_row_fact = o.m_row_fact;
        m_offsets = o.m_offsets;
        m_dia2off = o.m_dia2off;
        m_offsets_host = o.m_offsets_host;
        m_desc = o.m_desc;
        (const_cast<my_type *>(&o))->m_vec = NULL;
        return *this;
    }

    /// Run-table descriptor for the kernels (dev_memory_space only); built on
    /// first use from the host copy of the offsets.
    const cuvdia_desc *descriptor() const
    {
        static_assert(std::is_same<memory_space_type, dev_memory_space>::value,
                      "only device matrices carry a kernel descriptor");
        if (!m_desc) {
            cuvdia_desc *d = NULL;
            checkDiaCall(cuvdia_desc_create(&d, m_offsets_host.data(), m_num_dia, (int)this->h(), (int)this->w(),
                                            (int)m_stride, m_row_fact),
                         "cuvdia_desc_create");
            m_desc.reset(d, [](cuvdia_desc *p) { (void)hipDeviceSynchronize(); (void)cuvdia_desc_destroy(p); });
        }
        return m_desc.get();
    }

  private:
    void store_offsets(const std::vector<int> &v)
    {
        cuvAssert(v.size() <= m_offsets.size());
        std::copy(v.begin(), v.end(), m_offsets_host.begin());
        detail::copy<int, memory_space_type, host_memory_space>(m_offsets.ptr(), m_offsets_host.data(),
                                                                m_offsets_host.size());
        rebuild_map();
    }
    void rebuild_map()
    {
        m_dia2off.clear();
        for (unsigned int i = 0; i < m_offsets_host.size(); ++i) m_dia2off[m_offsets_host[i]] = i;
        m_desc.reset();
    }
};

}  // namespace cuv

namespace std {
template <class V, class T, class I>
ostream &operator<<(ostream &o, const cuv::dia_matrix<V, T, I> &w2)
{
    o << "Dia-Matrix: " << endl;
    for (I i = 0; i < w2.h(); i++) {
        for (I j = 0; j < w2.w(); j++) o << w2(i, j) << " ";
        o << endl;
    }
    o << endl;
    return o;
}
}  // namespace std
#endif
