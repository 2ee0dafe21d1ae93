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

}  // namespace kvt

struct kvt_block_lists {
  std::vector<kvt::RunList> tensors;
};

#endif  // KVT_INTERNAL_H_
