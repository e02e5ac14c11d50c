// The entry points of the quantised (GGUF) kernels for a build of the library that holds the dense-weight kernels only (`make dense`: libpipeinfer_amd_dense.so — a model
// described by config.json + safetensors needs nothing else, and the quantised mat-vec / matrix-core / attention kernels are most of a full build's compile time).
// Every one of them fails loudly: a GGUF model loaded through this build cannot decode.
#include "ops_common.h"

#include <climits>

static int absent(const char * what) { pi_set_error("%s: this library was built with the dense-weight kernels only (make -C pipeinfer_amd/csrc builds the full one)", what); return -1; }

int pi_mmq_min_nt() { return INT_MAX; }
int pi_mmq_max_nt() { return 0; }
int pi_mmq_step(int, int n_tok, int64_t) { return n_tok; }

extern "C" int pi_op_mmq_min_tokens(void) { return INT_MAX; }
extern "C" int pi_op_mul_mat_reserve(void) { return 0; }
extern "C" int pi_op_mul_mat_multi(int, const pi_weight * const *, const void *, int, float * const *, const float * const *, void *) { return absent("pi_op_mul_mat_multi"); }
extern "C" int pi_op_mul_mat(const pi_weight *, const void *, int, float *, const float *, void *) { return absent("pi_op_mul_mat"); }
extern "C" int pi_op_mul_mat_qkv_rope_ok(const pi_weight *, const pi_weight *, const pi_weight *, int, int) { return 0; }
extern "C" int pi_op_mul_mat_qkv_rope(const pi_weight *, const pi_weight *, const pi_weight *, const void *, int, const int32_t *, const void *, int, int, int, int, const int32_t *, uint16_t *, uint16_t *, uint16_t *,
                                      void *) { return absent("pi_op_mul_mat_qkv_rope"); }
extern "C" int pi_op_attention_max_cells(void) { return 0; }
extern "C" int pi_op_attention_reserve(int, int) { return absent("pi_op_attention_reserve"); }
extern "C" int pi_op_attention(const uint16_t *, const uint16_t *, const uint16_t *, const uint32_t *, int, int, int, int, int, float *, const int32_t *, void *) { return absent("pi_op_attention"); }
extern "C" int pi_op_attention_ex(const uint16_t *, const uint16_t *, const uint16_t *, const uint32_t *, int, int, int, int, int, float *, const int32_t *, int, void *) { return absent("pi_op_attention_ex"); }
extern "C" void pi_alibi_slopes(int n_head, float, float * out) { for (int i = 0; i < n_head; i++) out[i] = 0.0f; }
extern "C" int pi_op_attention_alibi(const uint16_t *, const uint16_t *, const uint16_t *, const uint32_t *, int, int, int, int, int, float *, const int32_t *, int, const float *, void *) { return absent("pi_op_attention_alibi"); }
