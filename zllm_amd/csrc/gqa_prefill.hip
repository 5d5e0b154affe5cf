#include "../../include/zllm_attn.h"
#include "kernels.hpp"
extern "C" {
uint64_t zllm_attn_gqa_prefill_workspace_bytes(const zllm_gqa_prefill_args*) { return 0; }
int zllm_attn_gqa_prefill_chunk(const zllm_gqa_prefill_args*, zllm_stream_t) { return -3; }
}
