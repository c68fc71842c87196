// Builds the DIA pattern of a locally connected layer.
//
// Mirrors filter_factory::get_dia of the reference
// (src/cuv/basics/filter_factory.hpp:43-76): an fs x fs window on a px x py
// map, input_maps -> output_maps, gives fs*fs*(output_maps + input_maps - 1)
// diagonals at offsets i*px + j + m*px*py, shifted so the window is centred
// and the first input map lines up.
#ifndef __FILTER_FACTORY_HPP__
#define __FILTER_FACTORY_HPP__

#include <algorithm>
#include <vector>

#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/tensor.hpp>

namespace cuv {

template <class T, class M, class I = unsigned int>
class filter_factory {
  public:
    typedef T value_type;
    typedef M memory_space;
    typedef I index_type;

    filter_factory(int px, int py, int fs, int input_maps, int output_maps)
        : m_px(px), m_py(py), m_fs(fs), m_input_maps(input_maps), m_output_maps(output_maps), m_dias_per_filter(0)
    {
    }

    /// Offsets only, in table order.
    std::vector<int> offsets() const
    {
        std::vector<int> off;
        for (int m = 0; m < m_output_maps + m_input_maps - 1; m++)
            for (int i = 0; i < m_fs; i++)
                for (int j = 0; j < m_fs; j++) off.push_back(i * m_px + j + m * m_px * m_py);
        const int shift = -(m_px + 1) * (m_fs / 2) - (m_input_maps - 1) * m_px * m_py;
        for (size_t i = 0; i < off.size(); i++) off[i] += shift;
        return off;
    }

    /// The weights that feed column `filternumber`, per input map: a new
    /// (fs*fs) x input_maps row-major tensor (caller owns it) whose flat entry
    /// map*fs*fs + k is the k-th stored element, rows ascending, of that
    /// column among the rows of input map `map`; filling stops when the
    /// tensor is full.  This is what src/cuv/basics/filter_factory.hpp:22-41
    /// sets out to do; its own text indexes the result pointer rather than
    /// the tensor, so there is no reference output to compare with.
    template <class M2>
    tensor<T, M, row_major> *extract_filter(const dia_matrix<T, M2, I> &dia, unsigned int filternumber)
    {
        const unsigned int fs2 = (unsigned int)(m_fs * m_fs);
        tensor<T, M, row_major> *mat = new tensor<T, M, row_major>(extents[fs2][m_input_maps]);
        const unsigned int total = mat->size();
        for (unsigned int k = 0; k < total; ++k) (*mat)[k] = (T)0;
        const unsigned int map_size = dia.h() / m_input_maps;
        for (unsigned int map_num = 0; map_num < (unsigned int)m_input_maps; map_num++) {
            unsigned int fi = 0;
            for (unsigned int i = 0; i < map_size; ++i) {
                const unsigned int row = i + map_num * map_size;
                if (!dia.has(row, filternumber)) continue;
                (*mat)[map_num * fs2 + fi++] = dia(row, filternumber);
                if (map_num * fs2 + fi >= total) break;
            }
        }
        return mat;
    }

    /// A new, value-uninitialised DIA matrix with that pattern (caller owns it).
    dia_matrix<T, M, I> *get_dia()
    {
        const std::vector<int> off = offsets();
        m_dias_per_filter = m_fs * m_fs;
        dia_matrix<T, M, I> *tp = new dia_matrix<T, M, I>(
            m_px * m_py * m_input_maps, m_px * m_py * m_output_maps, (int)off.size(),
            std::max(m_px * m_py * m_output_maps, m_px * m_py * m_input_maps));
        tp->set_offsets(off);
        return tp;
    }

  private:
    int m_px, m_py, m_fs, m_input_maps, m_output_maps;
    int m_dias_per_filter;
};

}  // namespace cuv
#endif
