// Owning device arrays for callers and tests (core/device_mdarray.hpp:127-183 in
// the reference): allocation on construction, release on destruction, view().
#pragma once

#include <utility>

#include <raft/core/device_mdspan.hpp>
#include <raft/core/resource/cuda_stream.hpp>

namespace raft {

template <typename ElementType, typename Extents, typename LayoutPolicy = layout_c_contiguous>
class device_mdarray {
 public:
  using view_type       = device_mdspan<ElementType, Extents, LayoutPolicy>;
  using const_view_type = device_mdspan<const ElementType, Extents, LayoutPolicy>;
  using index_type      = typename Extents::index_type;

  device_mdarray(resources const& res, Extents ext) : ext_(ext), stream_(res.get_stream())
  {
    size_t n = 1;
    for (size_t i = 0; i < Extents::rank(); ++i)
      n *= static_cast<size_t>(ext.extent(i));
    count_ = n;
    if (n > 0) RAFT_HIP_TRY(hipMalloc(reinterpret_cast<void**>(&ptr_), n * sizeof(ElementType)));
  }
  device_mdarray(device_mdarray&& o) noexcept
    : ptr_(std::exchange(o.ptr_, nullptr)), ext_(o.ext_), count_(o.count_), stream_(o.stream_)
  {
  }
  device_mdarray(const device_mdarray&)            = delete;
  device_mdarray& operator=(const device_mdarray&) = delete;
  ~device_mdarray()
  {
    if (ptr_ != nullptr) {
      (void)hipStreamSynchronize(stream_);
      (void)hipFree(ptr_);
    }
  }

  ElementType* data_handle() { return ptr_; }
  const ElementType* data_handle() const { return ptr_; }
  size_t size() const { return count_; }
  index_type extent(size_t i) const { return ext_.extent(i); }
  view_type view() { return view_type{ptr_, ext_}; }
  const_view_type view() const { return const_view_type{ptr_, ext_}; }

 private:
  ElementType* ptr_ = nullptr;
  Extents ext_{};
  size_t count_ = 0;
  hipStream_t stream_{};
};

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using device_matrix = device_mdarray<ElementType, matrix_extent<IndexType>, LayoutPolicy>;
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
using device_vector = device_mdarray<ElementType, vector_extent<IndexType>, LayoutPolicy>;
template <typename ElementType, typename IndexType = int>
using device_scalar = device_mdarray<ElementType, scalar_extent<IndexType>>;

template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
auto make_device_matrix(resources const& res, IndexType n_rows, IndexType n_cols)
{
  return device_matrix<ElementType, IndexType, LayoutPolicy>(
    res, matrix_extent<IndexType>{n_rows, n_cols});
}
template <typename ElementType, typename IndexType = int, typename LayoutPolicy = layout_c_contiguous>
auto make_device_vector(resources const& res, IndexType n)
{
  return device_vector<ElementType, IndexType, LayoutPolicy>(res, vector_extent<IndexType>{n});
}
template <typename ElementType, typename IndexType = int>
auto make_device_scalar(resources const& res)
{
  return device_scalar<ElementType, IndexType>(res, scalar_extent<IndexType>{});
}

}  // namespace raft
