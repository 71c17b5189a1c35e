// Number of set bits among the first max_len bits of a packed bit array
// (util/detail/popc.cuh:27-65 in the reference): a coalesced reduction over the words,
// seen as an N x 1 column-major matrix, whose main_op counts the bits of a word and masks
// the last word by its index.  The functor is a device lambda: compile with hipcc.
#pragma once

#include <raft/core/device_mdspan.hpp>
#include <raft/core/host_mdspan.hpp>
#include <raft/core/resources.hpp>
#include <raft/linalg/coalesced_reduction.cuh>

namespace raft::detail {

template <typename value_t, typename index_t>
void popc(const raft::resources& res,
          device_vector_view<const value_t, index_t> values,
          raft::host_scalar_view<const index_t, index_t> max_len,
          raft::device_scalar_view<index_t> counter)
{
  const index_t n_words = static_cast<index_t>(values.size());
  auto words = raft::make_device_matrix_view<const value_t, index_t, raft::col_major>(
    values.data_handle(), n_words, index_t{1});
  auto total = raft::make_device_vector_view<index_t, index_t>(counter.data_handle(), index_t{1});

  constexpr index_t bits_per_word = sizeof(value_t) * 8;
  const value_t live_bits         = static_cast<value_t>(max_len[0] % bits_per_word);
  // all ones when the last word is fully used
  const value_t last_mask =
    live_bits ? static_cast<value_t>((value_t{1} << live_bits) - value_t{1}) : static_cast<value_t>(~value_t{0});
  raft::linalg::coalesced_reduction(
    res, words, total, index_t{0}, false,
    [last_mask, n_words] __device__(value_t word, index_t i) {
      const value_t w = i == n_words - 1 ? static_cast<value_t>(word & last_mask) : word;
      if constexpr (sizeof(value_t) == 8) {
        return static_cast<index_t>(__popcll(static_cast<unsigned long long>(w)));
      } else {
        return static_cast<index_t>(__popc(static_cast<unsigned int>(w)));
      }
    });
}

}  // namespace raft::detail
