#include "da_mla.h"
namespace da {
bool mla_supported(size_t, size_t, int) { return false; }
int mla_heads_per_group(int) { return 1; }
int mla_rows_per_trip() { return 64; }
hipError_t launch_mla(const SweepParams&, bool, int, dim3, hipStream_t) { return hipErrorNotSupported; }
}  // namespace da
