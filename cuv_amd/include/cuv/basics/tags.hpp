// Memory-space and layout tags (src/cuv/basics/tags.hpp:13-20,
// src/cuv/basics/memory.hpp:32-36 of the reference).
#ifndef __CUV_TAGS_HPP__
#define __CUV_TAGS_HPP__
namespace cuv {
struct host_memory_space {};
struct dev_memory_space {};
struct row_major {};
struct column_major {};
}  // namespace cuv
#endif
