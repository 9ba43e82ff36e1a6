// Launch shapes and store policies of the shipped kernels, chosen by measurement on MI355X
// (Llama-3-8B and 70B decoder layers at world sizes 8 and 64, and a 2000-tensor ragged table;
// random data, the kernels of a step back to back: all-zero buffers run up to 10 % faster than
// any other content on this memory system and must not be used for tuning).
#pragma once
namespace yafsdp {

// ---- flat kernels (one contiguous range -> one contiguous range) -----------------------------
// workgroup size and units (8 elements) per lane per tile; loads are non-temporal.  With non-temporal stores the
// shapes 128 x 1, 128 x 2, 256 x 2 and 512 x 1 stay within 2 % of this one on 872-MB copies (135-145 us against 138)
// and are 1-4 % slower on the post-reduce of a 27 M-element shard (42.3-43.5 us against 41.9).  The byte kernel
// needs at least 128 lanes (workgroup 0 copies up to 127 leading bytes, one per lane).
constexpr int kFlatBlock = 256;
constexpr int kFlatUnroll = 1;
constexpr bool kFlatNtLoad = true;
// the post-reduce that also sums squares keeps tiles of 4096 elements: one partial sum per tile is part of its
// interface (yafsdp_post_reduce_sumsq_count), and the order of the additions must not move with the flat tuning
constexpr int kPostSumsqBlock = 256;
constexpr int kPostSumsqUnroll = 2;

// ---- table kernels (gather-in / scatter-out): a tile is block * unroll * 8 elements ----------
// Tiles of 1-2 K elements (2-4 KiB of bf16) in workgroups of one or two waves are the fastest for both kernels;
// larger workgroups lose 3-10 %.  Between the two, one wave per workgroup wins by 0.4 % on a 218 M-element buffer
// and two waves win by 2.8 % on an 856 M-element buffer (half as many workgroups to dispatch), so the tile size is
// chosen per table from its padded size.
constexpr int kTableBlockSmall = 64;
constexpr int kTableBlockLarge = 128;
constexpr int kTableLargeThresholdLog2 = 28;  // padded size above 2^28 elements: the larger workgroup
constexpr int kGatherUnroll = 2;              // units per lane of a gather-in tile (tiles of the flat buffer)
// scatter-out picks its tile per table (scatter_shape_for): one wave with ONE unit per lane (512-element tiles)
// when every tensor starts on a 128-byte line of the flat buffer, as the tensors of a transformer layer do
// (8B layer: 137.5 -> 133 us, 70B layer: 534 -> 517 us against two units per lane), and the gather-in shape
// otherwise (on a 1427-tensor table at odd offsets the short tiles lose 9 %: every tile then reads one more
// cache line than it writes, and shorter tiles make that line a larger share).
constexpr int kScatterShortUnroll = 1;
// Every load of the path is non-temporal: nothing enters the memory-side cache but what the store policy puts
// there.  (On the long scatter-out tile ordinary loads let the L2 keep the line that neighbouring tiles share and
// are 0.5-0.7 % faster by themselves, but what they read evicts the written-through end of the reduce buffer.)
constexpr bool kTableNtLoad = true;

// ---- store policy ---------------------------------------------------------------------------------
// A kernel stores non-temporal (ST_NT: the L2s keep the written lines and evict them as they fill) or
// write-through (ST_WT: the lines go to the memory side as they are produced and stay in its 256-MB cache until
// later traffic evicts them).  Which megabytes of a kernel's output write through is a run-time choice per kind of
// kernel (YAFSDP_OPT_*_TAIL_MB): always the END of the output, because a kernel whose last stores wrote through
// ends with clean L2s.  What write-through data is worth depends on whether it is still in that cache when its
// buffer is touched again, which only the caller knows.  The defaults below are the cache-neutral ones: every
// store non-temporal except the last 64 MB of the reduce buffer, which is the buffer a training run comes back to
// soonest (one gradient buffer shared by all parameter groups) and which measured as the best setting with two,
// three and four sets of buffers taking turns.  A caller that rewrites ONE set of buffers in a loop gains 2-4 %
// from writing through everywhere in the flat kernels and a 96-MB tail (policy "single_set" of the Python layer).
constexpr int kFlatStorePolicy = 2;     // ST_WT kernels; the tail option decides per tile
constexpr int kGatherStorePolicy = 1;   // ST_NT kernels whose tail tiles switch to ST_WT
constexpr int kScatterStorePolicy = 1;
constexpr int kGatherTailWriteThroughMb = 64;      // default of YAFSDP_OPT_GATHER_TAIL_MB
constexpr int kScatterTailWriteThroughMb = 0;      // default of YAFSDP_OPT_SCATTER_TAIL_MB
constexpr int kFlatTailWriteThroughMb = 0;         // default of YAFSDP_OPT_FLAT_TAIL_MB
constexpr int kPostReduceTailWriteThroughMb = 0;   // default of YAFSDP_OPT_POST_REDUCE_TAIL_MB

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

// ---- optimizer-side passes: a tile is block * unroll quads (4 elements each) ---------------------
constexpr int kFillBlock = 256;
constexpr int kFillUnroll = 1;    // 16-byte stores per lane per tile
constexpr int kScaleBlock = 256;
constexpr int kScaleUnroll = 2;   // (a mover without arithmetic runs this in-place mix at 34.2-37.0 us over twelve shapes; 36.7-36.9 us here)
constexpr int kSumsqBlock = 512;
constexpr int kSumsqUnroll = 4;
constexpr int kAdamBlock = 128;
constexpr int kAdamUnroll = 2;
constexpr bool kOptNtLoad = true;
constexpr bool kOptNtStore = true;
// An AdamW pass with a write-through tail gains 6 % when it visits the same shard again and again and loses 2 %
// over four shards in rotation (each is visited once per optimizer step): the optimizer kernels store non-temporal.
constexpr int kAdamStorePolicy = 1;

// ---- fan-out / fan-in: a tile is block * unroll units (fan-out) or quads (fan-in) --------------
// With 8 destinations the fan-out is 80 % stores.  Write-through stores make the kernel itself 5 % faster, but the
// kernel that runs after it pays three times that, so the stores stay non-temporal.  One pass over the source for
// all destinations: two passes of four take 115 us against 98.
constexpr int kFanOutBlock = 64;
constexpr int kFanOutUnroll = 1;
constexpr int kFanOutStorePolicy = 1;
constexpr int kFanInBlock = 64;
constexpr int kFanInUnroll = 1;

// workgroups (= partial sums) of the sum-of-squares pass; the workspace holds one double each
constexpr int kSumsqMaxPartials = 16384;
// default grid cap in workgroups per compute unit.  One workgroup per tile (no cap reached) beats a persistent
// grid-stride grid by 5-10 % on every kernel of the path, so the cap is far above any tile count of interest.
constexpr int kFlatBlocksPerCu = 4096;
constexpr int kTableBlocksPerCu = 4096;
}  // namespace yafsdp
