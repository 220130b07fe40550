// The head-dim-64 instantiation of the 64-row-per-wave attention kernels (attn_w64_tile<64, .>), as a
// translation unit of its own so that it compiles beside the head-dim-128 one: see the end of
// attention.hip.
#define FLUX_ATTN_W64_D64_UNIT
#include "attention.hip"
