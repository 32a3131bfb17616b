// Argument block shared by the routed-projection kernels (streaming rows kernel for decode,
// MFMA tile kernel for prefill) and their launcher.
#pragma once

#include "plan.h"
#include "../../include/mfq_amd.h"

namespace mfq_amd {

constexpr int kMaxPoolsPerTensor = 12;
constexpr int kPrefillTileM = 128;     // pairs per prefill tile of the plan
constexpr int kPrefillTileN = 64;      // output rows per block of the exact prefill kernel
constexpr int kRowsBlockRows = 64;     // output rows per decode block

// A projection over routed pairs: out[pair, slot, row] = W_slot[expert(pair)][row, :] . in[pair or token, :]
struct RowsArgs {
    const mfq_amd_projection* pools;   // device array, all slots
    const int32_t* expert_pool;        // [slots][experts] index into pools, -1 = absent
    const ExpertInfo* expert_info;     // [slots][experts] resolved pool, local index and class; null: expert_pool and pool_class serve
    const int32_t* pool_class;         // [pools] kernel class (| kPoolExactOnly)
    const int32_t* items;              // [slots][experts]
    const PlanItem* item_info;         // [slots][experts]
    const PairItem* pair_items;        // [slots][pairs]
    int32_t pairs;
    const int32_t* class_offsets;      // [slots][kClassSlots]
    const int32_t* tile_items;         // [slots][tile_capacity]
    const int32_t* tile_offsets;       // [slots][kClassSlots]
    const int32_t* expert_bounds;      // [experts + 1]
    const int32_t* ids_dst;            // [pairs]
    const void* in;                    // activations
    const uint32_t* in_packed;         // the same rows in the packed form of the streaming kernels, or null
    int64_t in_packed_stride;          // dwords between packed rows
    const uint16_t* in_tiles;          // the same rows as fp16 in the pair order of the weight classes (tile kernel), or null
    int64_t in_tiles_layout_stride;    // halves between the copies in the four pair layouts; 0: rows are in the order their consumer needs
    const uint8_t* in_fp8;             // block-scaled MFMA kernel: the activation rows as E4M3 terms, [row][terms][in_width] bytes
    const uint8_t* in_fp8_scales;      // their E8M0 block scales, [row][terms][in_width / 32]
    int32_t in_fp8_terms;              // 2 (bf16 source) or 3 (fp16 source): the terms add up to the source exactly
    int32_t skip_mxfp4;                // streaming tile kernel: leave MXFP4 tiles to the block-scaled MFMA kernel
    const uint16_t* gu;                // streaming decode kernel, down projection: gate/up outputs f16 [pair][2][in_width]; the block
                                       // computes hidden = swiglu(gate, up) of its pair itself.  Null: activations come from in / in_packed
    const uint16_t* sigmoid;           // the sigmoid table swiglu uses (gu != null)
    float swiglu_limit;
    uint16_t* out;                     // fp16
    int64_t out_pair_stride;           // halves between consecutive pairs
    int64_t out_slot_stride;           // halves between the outputs of consecutive slots of one pair
    int32_t in_dtype, in_per_pair, in_width, in_vector_ok;
    int32_t experts, top_k, tile_capacity;
    int32_t slot_base;                 // first slot of this launch; blockIdx.z adds to it
    int32_t out_rows;
    int32_t rows_per_block;            // streaming kernel: output rows per block, a multiple of rows_fast_min_block()
    int32_t exact_only;                // exact kernel: 1 = only items whose pool is marked kPoolExactOnly
    int32_t tile_slots;                // streaming tile kernel: slots of the launch (set by its launcher)
    int32_t grouped;                   // streaming rows kernel: pair_items carry group sizes (PlanExtras::group_pairs): a block
                                       // per group of up to kGroupPairs pairs of one expert
};

// True when the streaming fast path serves rows of this width and activation type.
bool rows_fast_geometry(int in_width, int in_dtype);
// Smallest rows_per_block (and its granularity) of the streaming kernel for rows of this width.
int rows_fast_min_block(int in_width);
// True when the pool itself qualifies for the fast path (its class is a fast class and its layout regular).
bool pool_fast_layout(const mfq_amd_projection& p);
// Exact decoders, one launch per kernel class that `present` marks; max_items[c] bounds the grid of class c.
// With args.exact_only set, only items of pools marked kPoolExactOnly are processed.
void launch_rows_exact(const RowsArgs& args, int slots, const int* present, const int* max_items, hipStream_t stream);
// Streaming fast path, one launch for every class and one block row per routed pair; `nvq` tells
// whether any pool needs the NVQ lookup tables.  Pairs of pools marked kPoolExactOnly are skipped.
void launch_rows_fast(const RowsArgs& args, int slots, bool nvq, hipStream_t stream);
// Prefill on the exact decoders, one launch per class; with args.exact_only set, only tiles of pools marked kPoolExactOnly.
void launch_rows_prefill(const RowsArgs& args, int slots, const int* present, const int* max_tiles, hipStream_t stream);
// True when the streaming MFMA tile kernel serves rows of this width, activation type and alignment.
bool tiles_fast_geometry(int in_width, int in_dtype, int in_vector_ok);
// Whether the tile kernel can take the rows as packed fp16 copies (RowsArgs::in_tiles): whole steps of 128 columns and
// a copy of less than 4 GB.
bool tiles_packed_geometry(int in_width, int64_t in_rows);
// Streaming MFMA tile kernel, one launch for every class; max_tiles bounds the tiles of a slot.
// Tiles of pools marked kPoolExactOnly are skipped.
void launch_tiles_fast(const RowsArgs& args, int slots, int max_tiles, bool nvq, hipStream_t stream);
// MXFP4 tiles on the block-scaled MFMA of gfx950 (fp4 weights with their E8M0 scales straight from memory, activations as
// E4M3 terms): the tiles of class K_MXFP4 of the plan; other tiles are skipped.
void launch_tiles_mx_scaled(const RowsArgs& args, int slots, int max_tiles, hipStream_t stream);
// dst[row][terms][width] E4M3 bytes and scales[row][terms][width / 32] E8M0 bytes of src[row][width] (fp16 or bf16);
// the terms of a block add up to the source values exactly (2 terms for bf16, 3 for fp16).
void launch_fp8_split(const void* src, int dtype, int rows, int width, int terms, uint8_t* dst, uint8_t* scales, hipStream_t stream);
// Pair layout (0..3) in which the streaming tile kernel reads the activations of a pool of this class.
int tile_layout_of_class(int cls);
// SwiGLU whose output rows are in the pair order their down projection reads (down_info: [experts]).
void launch_swiglu_tiles(const uint16_t* gate, const uint16_t* up, int64_t gate_stride, int inner, int pairs, float limit,
                         const uint16_t* table, const int32_t* ids, const ExpertInfo* down_info, int experts, uint16_t* hidden,
                         hipStream_t stream);

}  // namespace mfq_amd
