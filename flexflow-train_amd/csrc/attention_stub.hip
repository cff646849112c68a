// placeholder until attention.hip lands
#include "ffk_common.h"
using namespace ffk;
extern "C" int ffk_attention_forward(ffk_stream_t, int, ffk_attention_desc_t const *, void const *, void const *, void const *, void *, float *) { return fail(FFK_ERR_UNSUPPORTED, "attention_forward: not built yet"); }
extern "C" int ffk_attention_backward(ffk_stream_t, int, ffk_attention_desc_t const *, void const *, void const *, void const *, void const *, void const *, float const *, float *, void *, void *, void *) { return fail(FFK_ERR_UNSUPPORTED, "attention_backward: not built yet"); }
extern "C" size_t ffk_mha_weight_elements(ffk_mha_desc_t const *) { return 0; }
extern "C" size_t ffk_mha_reserve_bytes(ffk_mha_desc_t const *, int) { return 0; }
extern "C" int ffk_mha_forward(ffk_stream_t, int, ffk_mha_desc_t const *, void const *, void const *, void const *, void const *, void *, void *, size_t) { return fail(FFK_ERR_UNSUPPORTED, "mha_forward: not built yet"); }
extern "C" int ffk_mha_backward(ffk_stream_t, int, ffk_mha_desc_t const *, void const *, void *, void const *, void *, void const *, void *, void const *, void *, void const *, void *, size_t, int) { return fail(FFK_ERR_UNSUPPORTED, "mha_backward: not built yet"); }
