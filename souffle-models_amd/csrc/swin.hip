// placeholder until the Swin kernels land: every entry point reports "unsupported"
#include "host_util.hpp"
using namespace souffle;
extern "C" size_t souffle_swin_workspace_bytes(const souffle_swin_cfg *) { return 0; }
extern "C" int souffle_swin_block_pair_fused(const souffle_swin_cfg *, const souffle_swin_block_w *, const void *, void *, void *, size_t, souffle_stream_t) { return fail(SOUFFLE_ERR_UNSUPPORTED, "swin block pair is not built yet"); }
extern "C" int souffle_swin_index_maps(int, int, int, int, int32_t *, int32_t *, int32_t *, int32_t *) { return fail(SOUFFLE_ERR_UNSUPPORTED, "swin index maps are not built yet"); }
extern "C" int souffle_swin_ffn_fused(const void *, const void *, const void *, void *, void *, int, int, int, void *, size_t, souffle_stream_t) { return fail(SOUFFLE_ERR_UNSUPPORTED, "swin ffn is not built yet"); }
