// Route plan shared between the public route-plan entry point and the fused FFN.
#pragma once

#include "decode_classes.h"

#include "../../include/mfq_amd.h"

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mfq_amd {

constexpr int kPlanThreads = 1024;
constexpr int kPlanMaxExperts = 1024;
constexpr int kSlots = 3;                 // gate, up, down
constexpr int kClassSlots = dev::K_CLASS_COUNT + 1;

// One active expert of one slot, as the routed-projection kernels consume it (32 bytes).
struct PlanItem {
    int32_t expert;   // expert id
    int32_t pool;     // index into the pool array
    int32_t local;    // index of the expert inside its pool
    int32_t begin;    // first routed pair of the expert in ids_dst
    int32_t count;    // routed pairs of the expert
    int32_t cls;      // kernel class, plus kPoolExactOnly when the pool cannot take the streaming fast path
    int32_t reserved[2];
};
constexpr int kPoolExactOnly = 0x100;

// One routed pair of one slot, in the order of ids_dst (pairs of an expert are adjacent): what a block
// of the streaming kernel needs to start loading (16 bytes).
struct PairItem {
    int32_t pair;     // index of the pair (token * top_k + route), -1 behind the last routed pair
    int32_t pool;     // index into the pool array
    int32_t local;    // index of the expert inside its pool
    int32_t cls;      // kernel class (| kPoolExactOnly); with PlanExtras::group_pairs also, from bit kGroupCountShift, the
                      // number of pairs of the group this pair opens (1..kGroupPairs), 0 for the other pairs of a group
};
constexpr int kGroupPairs = 4;          // pairs of one expert that one block of the streaming rows kernel serves together
constexpr int kGroupCountShift = 16;

// What the plan needs to know about one expert of one slot, resolved once when the pools are fixed.
struct ExpertInfo {
    int32_t pool;     // index into the pool array, -1 = absent
    int32_t local;    // index inside the pool
    int32_t cls;      // kernel class of the pool (| kPoolExactOnly)
    int32_t reserved;
    int64_t bytes;    // packed bytes of the expert
};

// An ExpertInfo in one word: class word (9 bits) | pool << 9 (6 bits) | local << 15 (10 bits); all ones = absent.
constexpr uint32_t kExpertAbsent = 0xffffffffu;
inline uint32_t expert_word(int pool, int local, int cls_word) {
    return pool < 0 ? kExpertAbsent
                    : static_cast<uint32_t>(cls_word & 0x1ff) | (static_cast<uint32_t>(pool) << 9) | (static_cast<uint32_t>(local) << 15);
}

// Work lists the routed-projection kernels consume, all in device memory.
//   expert_pool[s][e]   index (into pools) of the pool that holds expert e in slot s, -1 = absent
//   items[s][i]         active experts of slot s sorted by (kernel class, expert id)
//   item_info[s][i]     the same list with pool, local index and pair range resolved
//   class_offsets[s][c] first item of class c in items[s]; [K_CLASS_COUNT] = number of active experts
//   tile_items[s][j]    prefill work: expert | (m_tile << 16), sorted by (class, expert, m_tile)
//   tile_offsets[s][c]  first tile of class c
struct PlanExtras {
    const mfq_amd_projection* pools;   // device array of every pool of every slot
    const int32_t* pool_class;         // [pools] kernel class (| kPoolExactOnly)
    const int64_t* pool_bytes;         // [pools] packed bytes of one expert of the pool
    int32_t slot_pool_begin[kSlots + 1];
    int32_t slots;                     // 1..3
    int32_t* expert_pool;              // [slots][experts], written unless expert_info is given
    const ExpertInfo* expert_info;     // [slots][experts] precomputed (pools never change between runs), or null
    const uint32_t* expert_words;      // [slots][experts] the same records in one word each (expert_word()), for pairs_only
    int32_t* items;                    // [slots][experts]
    PlanItem* item_info;               // [slots][experts] same order as items
    PairItem* pair_items;              // [slots][pairs]
    int32_t* class_offsets;            // [slots][kClassSlots]
    int32_t* tile_items;               // [slots][tile_capacity]
    int32_t* tile_offsets;             // [slots][kClassSlots]
    int64_t* touched_bytes;            // [1]
    int32_t* distinct;                 // [1]
    int32_t tile_capacity;
    int32_t prefill_tile_m;
    int32_t want_tiles;                // 0: tile_items / tile_offsets are not needed (decode)
    int32_t want_items;                // 0: items / item_info / class_offsets are not needed (no exact-kernel work)
    int32_t group_pairs;               // 1 (with pairs_only): neighbouring pairs of one expert form groups of up to kGroupPairs;
                                       // PairItem::cls carries the group sizes
    int32_t pairs_only;                // 1 (at most kPlanSortPairs pairs, expert_info given, no want_items / want_tiles):
                                       // only pair_items is produced, by the kernel that ranks the pairs directly;
                                       // none of counts, expert_bounds, ids_dst, items, touched_bytes, distinct written
};
constexpr int kPlanSortPairs = 512;

// Activation rows to bring into the packed form of the streaming kernels: one extra block per row.
struct PlanPack {
    const void* src;        // [rows][width] activations, null = nothing to pack
    uint32_t* dst;          // [rows][stride] packed rows
    int64_t stride;         // dwords between packed rows
    int32_t rows, width, dtype, vector_ok;
};

// Activation rows to copy as fp16 in the pair layouts of the streaming tile kernel (prefill): the spare blocks of the
// large plan kernel do it, kPlanThreads lane blocks of 32 columns each.
struct PlanTilePack {
    const void* src;        // [rows][width] activations (fp16 or bf16, 16-byte aligned rows), null = nothing to copy
    uint16_t* dst;          // [4][rows][width]: the copies, layout_stride halves apart
    int64_t layout_stride;
    int32_t rows, width, dtype;
    uint32_t layouts;       // bit l: layout l is wanted
    int64_t first_item;     // set by the launcher: the lane block (row * width / 32 + block) the launch's spare blocks start at
};

// Router logits to select the routes from inside the plan kernel (decode only), or logits == null.
struct PlanRoute {
    const void* logits;       // [tokens, experts]
    int32_t dtype, tokens, normalize;
    float norm_floor, scale;
    int32_t* ids_out;         // [tokens, top_k]
    float* weights_out;       // [tokens, top_k]
};

struct PlanArgs {
    const int32_t* ids;
    int32_t pairs, experts, tile_m;
    int32_t top_k;            // routes per token when ids is [tokens, top_k]; 0 = unknown
    int32_t* counts;          // [experts]
    int32_t* expert_bounds;   // [experts + 1]
    int32_t* tile_bounds;     // [experts + 1]
    int32_t* tile_experts;    // [pairs / tile_m + experts]
    int32_t* ids_dst;         // [pairs]
    int32_t* wave_base;       // [kPlanThreads / 64][experts] scratch, or null.  With it, a plan too large for the
                              // one-thread-per-pair kernel places its pairs with a second, multi-block kernel
    PlanExtras extras;        // extras.items == nullptr: plain route plan
    PlanPack pack;
    PlanTilePack tiles;
    int32_t lists_in_scatter;   // large plans (set by the launcher): the work lists are built by blocks of the scatter launch, one per slot
    PlanRoute route;
};

void launch_route_plan(const PlanArgs& args, hipStream_t stream);
// logits[tokens, experts] = x . router^T in fp32, columns added in ascending order per output.
void launch_router_logits(const void* x, int x_dtype, const void* router, int router_dtype, int tokens, int experts, int width,
                          float* logits, hipStream_t stream);
// touched_bytes[0] = packed bytes of the distinct experts `ids` names over the slots of expert_info; distinct[0] = their number.
void launch_touched_bytes(const int32_t* ids, int pairs, int experts, int slots, const ExpertInfo* expert_info,
                          int64_t* touched_bytes, int32_t* distinct, hipStream_t stream);

}  // namespace mfq_amd
