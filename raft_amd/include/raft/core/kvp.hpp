// raft::KeyValuePair: key first, then value, natural alignment — the layout the
// reduction library writes for arg-reductions (core/kvp.hpp:20-62 in the
// reference; the CUB conversions are dropped, there is no CUB here).
#pragma once

#include <raft/core/detail/macros.hpp>

namespace raft {

template <typename _Key, typename _Value>
struct KeyValuePair {
  typedef _Key Key;
  typedef _Value Value;

  Key key;
  Value value;

  KeyValuePair() = default;
  RAFT_INLINE_FUNCTION KeyValuePair(Key const& k, Value const& v) : key(k), value(v) {}

  RAFT_INLINE_FUNCTION bool operator!=(const KeyValuePair& b) const
  {
    return (value != b.value) || (key != b.key);
  }
  RAFT_INLINE_FUNCTION bool operator==(const KeyValuePair& b) const { return !(*this != b); }
  RAFT_INLINE_FUNCTION bool operator<(const KeyValuePair& b) const
  {
    return (key < b.key) || ((key == b.key) && value < b.value);
  }
  RAFT_INLINE_FUNCTION bool operator>(const KeyValuePair& b) const
  {
    return (key > b.key) || ((key == b.key) && value > b.value);
  }
};

}  // namespace raft
