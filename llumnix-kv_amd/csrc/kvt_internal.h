// Internal declarations shared by the host-side translation units of libkvt_hip.
#ifndef KVT_INTERNAL_H_
#define KVT_INTERNAL_H_

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "kvt_hip.h"

namespace kvt {

// Records the calling thread's error message and returns `code`.
int fail(int code, const std::string& msg);
void clear_error();

struct RangeError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct OverflowError : std::runtime_error {
  using std::runtime_error::runtime_error;
};
struct InvalidError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// Runs `body`, translating the library's internal exceptions into KVT_* codes.
template <class F>
int guarded(F&& body) {
  try {
    return body();
  } catch (const RangeError& e) {
    return fail(KVT_ERR_OUT_OF_RANGE, e.what());
  } catch (const OverflowError& e) {
    return fail(KVT_ERR_OVERFLOW, e.what());
  } catch (const InvalidError& e) {
    return fail(KVT_ERR_INVALID, e.what());
  } catch (const std::bad_alloc&) {
    return fail(KVT_ERR_INVALID, "out of host memory");
  } catch (const std::exception& e) {
    return fail(KVT_ERR_INVALID, e.what());
  }
}

typedef std::vector<kvt_ipc_block> RunList;

// Stable permutation that orders `keys` ascending: LSD radix sort on 11-bit
// digits, skipping digits that are constant over the input. Returns early with
// the identity when the keys are already ascending (the common case for a
// sender's list that was merged before). O(n) instead of O(n log n): the lists
// of a large batch hold tens of thousands of ranges.
void stable_order_by_key(const std::vector<uint64_t>& keys, std::vector<uint32_t>& order);

}  // namespace kvt

struct kvt_block_lists {
  std::vector<kvt::RunList> tensors;
};

struct kvt_run_lists {
  std::vector<std::vector<kvt_run>> tensors;
};

#endif  // KVT_INTERNAL_H_
