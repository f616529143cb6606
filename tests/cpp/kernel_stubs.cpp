// Stand-ins for the GPU entry points of the library in the host-only sanitizer builds: the engine
// refers to them, the host backend never calls them.
#include <cstdint>
#include <cstdio>

#define STUB(name) extern "C" int name(...) { fprintf(stderr, "kernel entry " #name " called in the host-only build\n"); return -1; }
STUB(moe_gate_logits)
STUB(moe_gate_logits_pair)
STUB(moe_topk)
STUB(moe_dispatch)
STUB(moe_dispatch_ws)
STUB(moe_route_decode)
STUB(moe_topk_dispatch)
STUB(moe_gate_topk_dispatch)
STUB(moe_decode_batch_int4_gate)
STUB(moe_experts_decode_int4)
STUB(moe_experts_decode_int4_publish)
STUB(moe_decode_token_int4)
STUB(moe_decode_token_int4_gate)
STUB(moe_decode_token_late_expert_int4)
STUB(moe_experts_decode_q4k)
STUB(moe_experts_prefill)
STUB(moe_experts_prefill_pieces)
STUB(moe_combine)
STUB(moe_combine_splits)
extern "C" int moe_decode_shared_splits(...) { return 1; }
extern "C" int moe_prefill_shared_splits(...) { return 1; }
extern "C" int64_t moe_prefill_workspace_bytes(...) { return 0; }
extern "C" int64_t moe_dispatch_workspace_bytes(...) { return 0; }
extern "C" int64_t moe_gate_ws_bytes(...) { return 64; }
extern "C" int64_t moe_gate_route_ws_bytes(...) { return 64; }
extern "C" int moe_decode_batch_int4_gate_fits(...) { return 0; }
