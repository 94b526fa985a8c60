// Entry points whose kernels are not written yet: they report hipErrorNotSupported.
#include "common.hpp"
#define NS return (int)hipErrorNotSupported
TA_EXPORT int thrust_amd_merge(void*, size_t*, const void*, uint64_t, const void*, uint64_t, void*, int, int, void*) { NS; }
TA_EXPORT int thrust_amd_merge_by_key(void*, size_t*, const void*, uint64_t, const void*, uint64_t, const void*, const void*, void*, void*, int, size_t, int, void*) { NS; }
