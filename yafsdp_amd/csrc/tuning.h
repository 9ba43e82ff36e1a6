// Launch shapes of the shipped kernels, chosen by measurement on MI355X
// (Llama-3-8B decoder layer at world size 8, and a 2000-tensor ragged table).
#pragma once
namespace yafsdp {
// flat kernels: workgroup size, units (8 elements) per lane per tile,
// non-temporal loads / stores
#ifndef YAFSDP_FLAT_BLOCK
#define YAFSDP_FLAT_BLOCK 256
#endif
#ifndef YAFSDP_FLAT_U
#define YAFSDP_FLAT_U 1
#endif
// issue priority the copy kernels' waves ask for (s_setprio, 0..3; 0 leaves the default)
#ifndef YAFSDP_WAVE_PRIO
#define YAFSDP_WAVE_PRIO 0
#endif
constexpr int kWavePrio = YAFSDP_WAVE_PRIO;
// store policy of whole tiles: 0 ordinary, 1 non-temporal, 2 write-through (see TileStore)
#ifndef YAFSDP_FLAT_STP
#define YAFSDP_FLAT_STP 2
#endif
#ifndef YAFSDP_TABLE_STP
#define YAFSDP_TABLE_STP 1
#endif
constexpr int kFlatBlock = YAFSDP_FLAT_BLOCK;
constexpr int kFlatUnroll = YAFSDP_FLAT_U;
// the post-reduce that also sums squares keeps tiles of 4096 elements: one partial sum per tile is part of its
// interface (yafsdp_post_reduce_sumsq_count), and the order of the additions must not move with the flat tuning
constexpr int kPostSumsqBlock = 256;
constexpr int kPostSumsqUnroll = 2;
#ifndef YAFSDP_FLAT_NTL
#define YAFSDP_FLAT_NTL true
#endif
constexpr bool kFlatNtLoad = YAFSDP_FLAT_NTL;
constexpr int kFlatStorePolicy = YAFSDP_FLAT_STP;
// gather-in / scatter-out: a tile is block * unroll * 8 elements.  Measured with
// non-zero data and the four kernels of a step running back to back: tiles of
// 1-2 K elements (2-4 KiB of bf16) in workgroups of one or two waves are the
// fastest for both kernels; larger workgroups lose 3-10 %.  Between the two,
// one wave per workgroup wins by 0.4 % on a 218 M-element buffer and two waves
// win by 2.8 % on an 856 M-element buffer (half as many workgroups to
// dispatch), so the tile size is chosen per table from its padded size.
// (All-zero buffers run up to 10 % faster than any other content on this memory
// system and must not be used for tuning.)
constexpr int kTableBlockSmall = 64;
#ifndef YAFSDP_TABLE_BLOCK_LARGE
#define YAFSDP_TABLE_BLOCK_LARGE 128
#endif
constexpr int kTableBlockLarge = YAFSDP_TABLE_BLOCK_LARGE;
constexpr int kTableLargeThresholdLog2 = 28;  // padded size above 2^28 elements: the larger workgroup
#ifndef YAFSDP_TABLE_U
#define YAFSDP_TABLE_U 2
#endif
#ifndef YAFSDP_GATHER_U
#define YAFSDP_GATHER_U YAFSDP_TABLE_U
#endif
constexpr int kGatherUnroll = YAFSDP_GATHER_U;    // units per lane of a gather-in tile (tiles of the flat buffer)
// scatter-out picks its tile per table (scatter_shape_for): one wave with ONE unit per lane (512-element tiles)
// when every tensor starts on a 128-byte line of the flat buffer, as the tensors of a transformer layer do
// (8B layer: 137.5 -> 133 us, 70B layer: 534 -> 517 us against two units per lane), and the gather-in shape
// otherwise (on a 1427-tensor table at odd offsets the short tiles lose 9 %: every tile then reads one more
// cache line than it writes, and shorter tiles make that line a larger share).
constexpr int kScatterShortUnroll = 1;
#ifndef YAFSDP_TABLE_NTL
#define YAFSDP_TABLE_NTL true
#endif
// 0: workgroup b handles tile b.  X > 0: workgroups are assumed to be dealt round-robin to X XCDs, and within every
// window of X * R tiles each XCD takes a run of R neighbouring tiles (tile = window + (b % X) * R + (b / X) % R), so
// that neighbouring tiles, which share a cache line on the side with odd offsets, meet in one L2.
#ifndef YAFSDP_TABLE_XCD
#define YAFSDP_TABLE_XCD 0
#endif
#ifndef YAFSDP_TABLE_XCD_RUN
#define YAFSDP_TABLE_XCD_RUN 8
#endif
constexpr int kTableXcd = YAFSDP_TABLE_XCD;
constexpr int kTableXcdRun = YAFSDP_TABLE_XCD_RUN;
constexpr bool kTableNtLoad = YAFSDP_TABLE_NTL;
// scatter-out reads the flat buffer with non-temporal loads on both tile shapes, like every other kernel.  On the
// long tile (tensors at odd offsets: every tile shares its first and last line with a neighbour) ordinary loads let
// the L2 keep the shared line and are 0.5-0.7 % faster by themselves (573-tensor table, copy-out as a launch of its
// own 107 -> 105 us), but what they read also passes through the memory-side cache and evicts the written-through
// end of the reduce buffer that the store policy below keeps there: with that tail the step of the 573-tensor group
// takes 0.2773 ms with ordinary loads and 0.2685 ms with non-temporal ones (0.2718 without any tail), that of the
// 1427-tensor group 0.4778 and 0.4727 ms (0.4742).  Ordinary loads in gather-in move time from one kernel of the step
// to the next without shortening the step (1427 tensors: copy-out 237 -> 232 us, reduce copy-in 230 -> 236 us).
#ifndef YAFSDP_SCATTER_LONG_NTL
#define YAFSDP_SCATTER_LONG_NTL true
#endif
constexpr bool scatter_nt_load(int unroll) {
  return unroll == 1 ? bool(YAFSDP_TABLE_NTL) : bool(YAFSDP_SCATTER_LONG_NTL);
}
#ifndef YAFSDP_GATHER_STP
#define YAFSDP_GATHER_STP YAFSDP_TABLE_STP
#endif
#ifndef YAFSDP_SCATTER_STP
#define YAFSDP_SCATTER_STP YAFSDP_TABLE_STP
#endif
// Store policy.  A kernel stores non-temporal (the L2s keep the written lines and evict them as they fill) or
// write-through (the lines go to the memory side as they are produced and stay in
// its 256-MB cache until later traffic evicts them).  Which megabytes of a kernel's output write through is a
// run-time choice per kind of kernel: always the END of the output (the last tiles of the flat buffer in gather-in,
// the tile slots of the last tensors in scatter-out, the last tiles of a flat pass), because a kernel whose last
// stores wrote through ends with clean L2s (its closing write-back finds no dirty line, 40 thousand otherwise).
// What write-through data is worth depends on whether it is still in that cache when its buffer is touched again:
// a later read is then served from there, and a later write overwrites it before it ever reached DRAM.
//  * One set of buffers rewritten step after step (a loop over one layer; a model with one parameter group): much of
//    what wrote through is found again.  Llama-3-8B layer, ms per step, megabytes of (flat kernels, post-reduce,
//    scatter-out tail, gather-in tail): (all, all, 0, 0) 0.3272; (all, all, 0, 64) 0.3239; (all, all, 0, 96) 0.3226,
//    the defaults below; (all, all, 0, 128) 0.3334; (all, all, 32, 56) 0.3200, but the reduce copy-in itself then
//    runs 135 us instead of 131.5 (it pays for the copy-out's lines); (all, all, 32, 96) 0.3295; (0, 0, 0, 0) 0.3309;
//    (0, 0, 0, 128) 0.3268.
//  * K sets of buffers taking turns, 2.2 GB of other traffic between two visits of a set: a set's written-through end
//    survives until its next visit if K of them fit the cache together, and costs (evictions of dirty lines in the
//    middle of other kernels) if they do not.  Gather-in tail alone, everything else non-temporal, same layer:
//    K=2: 0 MB 0.3317, 96 MB 0.3285, 128 MB 0.3277, 144 MB 0.3321; K=3: 0 MB 0.3323, 64 MB 0.3299, 85 MB 0.3294,
//    128 MB 0.3340; K=4: 0 MB 0.3339, 64 MB 0.3320, 85 MB 0.3359.  With (all, all, 32, 56): K=2 0.3329, K=3 0.3346,
//    K=4 0.3354 (write-through everywhere in the flat kernels already overfills the cache).  The reference shares ONE
//    gradient buffer among all parameter groups (and two gathered buffers), so the reduce buffer's end is what comes
//    round soonest: the policy that the fully_shard layer selects for models with several groups writes the last
//    128 MB of the reduce buffer through and nothing else (options at run time), which is also what a full pass over
//    35 groups measures as best, alone and next to GEMMs.
// An AdamW pass with a write-through tail gains 6 % when it visits the same shard again and again and loses 2 % over
// four shards in rotation (each is visited once per optimizer step): the optimizer kernels store non-temporal.
#ifndef YAFSDP_GATHER_TAIL_WT_MB
#define YAFSDP_GATHER_TAIL_WT_MB 96
#endif
#ifndef YAFSDP_SCATTER_TAIL_WT_MB
#define YAFSDP_SCATTER_TAIL_WT_MB 0
#endif
constexpr int kGatherTailWriteThroughMb = YAFSDP_GATHER_TAIL_WT_MB;    // default of YAFSDP_OPT_GATHER_TAIL_MB
constexpr int kScatterTailWriteThroughMb = YAFSDP_SCATTER_TAIL_WT_MB;  // default of YAFSDP_OPT_SCATTER_TAIL_MB
// The flat kernels write through everywhere by default (the option counts megabytes at the end of their output
// like the two above; 2^20 covers any buffer, 0 stores everything non-temporal).
#ifndef YAFSDP_FLAT_TAIL_WT_MB
#define YAFSDP_FLAT_TAIL_WT_MB (1 << 20)
#endif
constexpr int kFlatTailWriteThroughMb = YAFSDP_FLAT_TAIL_WT_MB;  // default of YAFSDP_OPT_FLAT_TAIL_MB
#ifndef YAFSDP_POST_REDUCE_TAIL_WT_MB
#define YAFSDP_POST_REDUCE_TAIL_WT_MB (1 << 20)
#endif
constexpr int kPostReduceTailWriteThroughMb = YAFSDP_POST_REDUCE_TAIL_WT_MB;  // of YAFSDP_OPT_POST_REDUCE_TAIL_MB
constexpr int kGatherStorePolicy = YAFSDP_GATHER_STP;
constexpr int kScatterStorePolicy = YAFSDP_SCATTER_STP;
inline int table_block_for(long long padded_elems, int threshold_log2) {
  return padded_elems > (1LL << threshold_log2) ? kTableBlockLarge : kTableBlockSmall;
}
inline long long gather_tile_elems(int block) { return (long long)block * kGatherUnroll * 8; }
struct ScatterShape { int block, unroll; };
// mode: 0 from the layout, 1 always the short tile, 2 never
inline ScatterShape scatter_shape_for(long long padded_elems, bool line_aligned, int threshold_log2, int mode) {
  if (mode == 1 || (mode == 0 && line_aligned)) return ScatterShape{kTableBlockSmall, kScatterShortUnroll};
  return ScatterShape{table_block_for(padded_elems, threshold_log2), kGatherUnroll};
}
inline long long scatter_tile_elems(ScatterShape s) { return (long long)s.block * s.unroll * 8; }
// optimizer-side passes: a tile is block * unroll quads (4 elements each)
#ifndef YAFSDP_FILL_BLOCK
#define YAFSDP_FILL_BLOCK 256
#endif
#ifndef YAFSDP_FILL_U
#define YAFSDP_FILL_U 1
#endif
#ifndef YAFSDP_SCALE_BLOCK
#define YAFSDP_SCALE_BLOCK 256
#endif
#ifndef YAFSDP_SCALE_U
#define YAFSDP_SCALE_U 2
#endif
#ifndef YAFSDP_SUMSQ_BLOCK
#define YAFSDP_SUMSQ_BLOCK 512
#endif
#ifndef YAFSDP_SUMSQ_U
#define YAFSDP_SUMSQ_U 4
#endif
#ifndef YAFSDP_ADAM_BLOCK
#define YAFSDP_ADAM_BLOCK 128
#endif
#ifndef YAFSDP_ADAM_U
#define YAFSDP_ADAM_U 2
#endif
constexpr int kFillBlock = YAFSDP_FILL_BLOCK;
constexpr int kFillUnroll = YAFSDP_FILL_U;    // 16-byte stores per lane per tile
constexpr int kScaleBlock = YAFSDP_SCALE_BLOCK;
constexpr int kScaleUnroll = YAFSDP_SCALE_U;
constexpr int kSumsqBlock = YAFSDP_SUMSQ_BLOCK;
constexpr int kSumsqUnroll = YAFSDP_SUMSQ_U;
constexpr int kAdamBlock = YAFSDP_ADAM_BLOCK;
constexpr int kAdamUnroll = YAFSDP_ADAM_U;
constexpr bool kOptNtLoad = true;
constexpr bool kOptNtStore = true;
// store policy of the fused Adam(W) pass (see TileStore)
#ifndef YAFSDP_ADAM_STP
#define YAFSDP_ADAM_STP 1
#endif
constexpr int kAdamStorePolicy = YAFSDP_ADAM_STP;
// fan-out: a tile is block * unroll units.  With 8 destinations the kernel is 80 % stores.  Write-through stores
// (see TileStore) with 256 lanes make the kernel itself 5 % faster (94.9 against 99.3 us on a 27 M-element shard),
// but the kernel that runs after it pays three times that (the fan-in of the same step: 94 -> 113 us), so the
// stores stay non-temporal.  One pass over the source for all destinations: two passes of four take 115 us.
// 256 lanes, two units per lane or a fully unrolled destination loop are level or slower (98 -> 99-108 us).
#ifndef YAFSDP_FANOUT_BLOCK
#define YAFSDP_FANOUT_BLOCK 64
#endif
#ifndef YAFSDP_FANOUT_U
#define YAFSDP_FANOUT_U 1
#endif
#ifndef YAFSDP_FANOUT_STP
#define YAFSDP_FANOUT_STP 1
#endif
// fan-in: a tile is block * unroll quads
#ifndef YAFSDP_FANIN_BLOCK
#define YAFSDP_FANIN_BLOCK 64
#endif
#ifndef YAFSDP_FANIN_U
#define YAFSDP_FANIN_U 1
#endif
constexpr int kFanOutBlock = YAFSDP_FANOUT_BLOCK;
constexpr int kFanOutUnroll = YAFSDP_FANOUT_U;
constexpr int kFanOutStorePolicy = YAFSDP_FANOUT_STP;
constexpr int kFanInBlock = YAFSDP_FANIN_BLOCK;
constexpr int kFanInUnroll = YAFSDP_FANIN_U;
// workgroups (= partial sums) of the sum-of-squares pass; the workspace holds one double each
constexpr int kSumsqMaxPartials = 16384;
// default grid cap in workgroups per compute unit.  Measured: one workgroup per
// tile (no cap reached) beats a persistent grid-stride grid by 5-10 % on every
// kernel of the path, so the cap is far above any tile count of interest.
constexpr int kFlatBlocksPerCu = 4096;
constexpr int kTableBlocksPerCu = 4096;
}  // namespace yafsdp
