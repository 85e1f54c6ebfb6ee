// How many queries a tile of each attention kernel's work list holds: the one place where these
// sizes are written.  The kernels include it; who makes the lists asks eng_attn_tile_sizes().
#pragma once

#define ATTN_TILE_QUERIES 16           // attn_tile (attention.hip): queries a block
#define ATTN_PREFILL_TILE_QUERIES 128  // attn_prefill (attention_prefill.hip): queries a block
