#include "common.hpp"
extern "C" {
size_t tango_qgemm_fwd_workspace(int64_t, int64_t, int64_t) { return 0; }
int tango_qgemm_fwd(float*, int64_t, const float*, int64_t, int8_t*, const float*, int64_t, int8_t*, const float*, float*, const float*, const float*, int64_t, int64_t, int64_t, int, void*, size_t, tango_stream_t) { return TANGO_ERR_UNSUPPORTED; }
int tango_qgemm_i8_nt(float*, int64_t, const int8_t*, int64_t, const int8_t*, int64_t, const float*, float*, const float*, const float*, int64_t, int64_t, int64_t, tango_stream_t) { return TANGO_ERR_UNSUPPORTED; }
int tango_qgemm_bwd_dx(float*, int64_t, const int8_t*, int64_t, const int8_t*, int64_t, const float*, const float*, int64_t, int64_t, int64_t, tango_stream_t) { return TANGO_ERR_UNSUPPORTED; }
size_t tango_qgemm_bwd_dw_workspace(int64_t, int64_t, int64_t) { return 0; }
int tango_qgemm_bwd_dw(float*, int64_t, const int8_t*, int64_t, const int8_t*, int64_t, const float*, const float*, int64_t, int64_t, int64_t, void*, size_t, tango_stream_t) { return TANGO_ERR_UNSUPPORTED; }
size_t tango_qgemm_legacy_workspace(int64_t, int64_t, int64_t) { return 0; }
int tango_qgemm_legacy(float*, const float*, const float*, int64_t, int64_t, int64_t, int, int, void*, size_t, tango_stream_t) { return TANGO_ERR_UNSUPPORTED; }
}
