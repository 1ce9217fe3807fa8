#include "common.hpp"
namespace smoe {
bool try_s2s_mfma(const S2SArgs&, int, hipStream_t, int&) { return false; }
bool try_xty_mfma(const XtYArgs&, int, hipStream_t, int&) { return false; }
}
