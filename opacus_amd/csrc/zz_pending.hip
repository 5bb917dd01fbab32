// Entry points declared in dpk.h whose kernels are still being written: they fail loudly.
#include "dpk_common.h"
#define PENDING(name) return dpk_fail(DPK_E_ARG, "%s: not implemented in this build", name)
extern "C" size_t dpk_embedding_workspace_bytes(int64_t, int64_t) { return 0; }
extern "C" int dpk_embedding_unique_pairs(const int64_t*, int64_t, int64_t, int64_t*, int64_t*, int64_t*, void*, size_t, dpk_stream_t) { PENDING("dpk_embedding_unique_pairs"); }
extern "C" int dpk_embedding_gs(const int64_t*, const void*, int, void*, int, int64_t, int64_t, int64_t, int64_t, float, void*, size_t, dpk_stream_t) { PENDING("dpk_embedding_gs"); }
extern "C" int dpk_embedding_ghost_norm(const int64_t*, const void*, int, float*, int64_t, int64_t, int64_t, float, void*, size_t, dpk_stream_t) { PENDING("dpk_embedding_ghost_norm"); }
extern "C" int dpk_group_norm_gs(const void*, const void*, int, void*, void*, int, int64_t, int64_t, int64_t, int64_t, float, float, dpk_stream_t) { PENDING("dpk_group_norm_gs"); }
extern "C" size_t dpk_rms_norm_gs_workspace_bytes(int64_t, int64_t, int64_t) { return 0; }
extern "C" int dpk_rms_norm_gs(const void*, const void*, int, void*, int, int64_t, int64_t, int64_t, float, float, void*, size_t, dpk_stream_t) { PENDING("dpk_rms_norm_gs"); }
