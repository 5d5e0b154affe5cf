#include "../../include/zllm_attn.h"
#include "kernels.hpp"
extern "C" {
uint64_t zllm_attn_mla_decode_workspace_bytes(const zllm_mla_decode_args*) { return 0; }
int zllm_attn_mla_decode(const zllm_mla_decode_args*, zllm_stream_t) { return -3; }
}
