// Entry points of the reference's GPU plugin that lie outside the batched
// signature path.  The reference's loader binds every symbol eagerly at import
// (pysiglib/load_siglib.py:113-130,165-182,420-641), so each one must exist; here
// they report "not implemented" with the generic runtime-error status instead of
// computing anything.
#include <cstdio>

extern "C" const char* cusig_last_error_message(void) noexcept;

namespace {
int not_implemented(const char* name) noexcept
{
    // the message buffer is owned by the API translation unit; writing through the
    // returned pointer keeps a single thread-local buffer for the whole library
    char* buf = const_cast<char*>(cusig_last_error_message());
    std::snprintf(buf, 4096, "%s is not implemented in this build (only the batched signature path is)", name);
    return 10;
}
}  // namespace

#define STUB_PAIR(name)                                                                              \
    extern "C" __attribute__((visibility("default"))) int name##_f(...) noexcept { return not_implemented(#name "_f"); } \
    extern "C" __attribute__((visibility("default"))) int name##_d(...) noexcept { return not_implemented(#name "_d"); }
#define STUB_ONE(name) \
    extern "C" __attribute__((visibility("default"))) int name(...) noexcept { return not_implemented(#name); }

STUB_PAIR(log_sig_combine_cuda)
STUB_PAIR(log_sig_from_path_cuda)
STUB_PAIR(log_sig_from_path_backprop_cuda)
STUB_PAIR(log_sig_combine_backprop_cuda)
STUB_PAIR(sig_kernel_cuda)
STUB_PAIR(sig_kernel_poly_cuda)
STUB_PAIR(sig_kernel_poly_backprop_cuda)
STUB_PAIR(branched_sig_kernel_cuda)
STUB_PAIR(sig_kernel_backprop_cuda)
STUB_PAIR(branched_sig_kernel_backprop_cuda)
STUB_PAIR(branched_sig_kernel_poly_cuda)
STUB_PAIR(branched_sig_kernel_poly_backprop_cuda)
STUB_PAIR(branched_sig_cuda)
STUB_PAIR(branched_sig_coef_cuda)
STUB_PAIR(branched_sig_coef_backprop_cuda)
STUB_PAIR(branched_sig_combine_cuda)
STUB_PAIR(branched_sig_to_log_sig_cuda)
STUB_PAIR(branched_sig_to_log_sig_backprop_cuda)
STUB_PAIR(branched_log_sig_join_cuda)
STUB_PAIR(branched_log_sig_join_backprop_cuda)
STUB_PAIR(branched_log_sig_from_path_cuda)
STUB_PAIR(branched_log_sig_from_path_backprop_cuda)
STUB_PAIR(branched_sig_combine_backprop_cuda)
STUB_PAIR(branched_sig_backprop_cuda)
STUB_PAIR(log_sig_join_cuda)
STUB_PAIR(log_sig_join_backprop_cuda)
STUB_PAIR(logsig_to_sig_cuda)
STUB_PAIR(logsig_to_sig_backprop_cuda)
STUB_ONE(set_cache_dir_cuda)
STUB_ONE(prepare_branched_sig_cuda)
STUB_ONE(prepare_branched_log_sig_cuda)
STUB_ONE(prepare_branched_sig_coef_cuda)
