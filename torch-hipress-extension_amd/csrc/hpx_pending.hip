// Entry points whose kernels are not written yet: they fail loudly.
#include "hpx_common.h"
#define PENDING(name) do { hpx::set_error(name ": not implemented"); return HPX_ERR_ARG; } while (0)
HPX_API int hpx_powersgd_encode1(int, const float* const*, const int64_t*, const float* const*, const float* const*, float* const*, float* const*, const int32_t*, const int32_t*, const int32_t*, hpx_stream_t) { PENDING("hpx_powersgd_encode1"); }
HPX_API int hpx_powersgd_encode2(int, float* const*, const float* const*, float* const*, const int32_t*, const int32_t*, const int32_t*, hpx_stream_t) { PENDING("hpx_powersgd_encode2"); }
HPX_API int hpx_powersgd_decode(int, const float* const*, const float* const*, float* const*, float* const*, float* const*, const int64_t*, const int32_t*, const int32_t*, const int32_t*, hpx_stream_t) { PENDING("hpx_powersgd_decode"); }
