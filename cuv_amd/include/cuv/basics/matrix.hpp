// Width/height base of the matrix types (src/cuv/basics/matrix.hpp:49-106 of
// the reference).
#ifndef __CUV_MATRIX_HPP__
#define __CUV_MATRIX_HPP__

#include <cuv/tools/cuv_general.hpp>

namespace cuv {

template <class __value_type, class __index_type>
class matrix {
  public:
    typedef __value_type value_type;
    typedef __index_type index_type;

  protected:
    index_type m_width;
    index_type m_height;

  public:
    matrix(const index_type &h, const index_type &w) : m_width(w), m_height(h) {}
    matrix(const matrix &m) : m_width(m.w()), m_height(m.h()) {}
    matrix &operator=(const matrix &m)
    {
        m_width = m.w();
        m_height = m.h();
        return *this;
    }
    virtual ~matrix() {}
    inline void resize(const index_type &h, const index_type &w)
    {
        cuvAssert(w * h == m_width * m_height);
        m_width = w;
        m_height = h;
    }
    inline index_type w() const { return m_width; }
    inline index_type h() const { return m_height; }
    inline index_type n() const { return w() * h(); }
};

}  // namespace cuv
#endif
