// Launch shapes of the shipped kernels, chosen by measurement on MI355X
// (Llama-3-8B decoder layer at world size 8, and a 2000-tensor ragged table).
#pragma once
namespace yafsdp {
// flat kernels: workgroup size, units (8 elements) per lane per tile,
// non-temporal loads / stores
constexpr int kFlatBlock = 256;
constexpr int kFlatUnroll = 2;
constexpr bool kFlatNtLoad = true;
constexpr bool kFlatNtStore = true;
// gather-in / scatter-out: a tile is block * unroll * 8 elements.  Measured with
// non-zero data and the four kernels of a step running back to back: tiles of
// 1-2 K elements (2-4 KiB of bf16) in workgroups of one or two waves are the
// fastest for both kernels (one wave x 2 units ahead by about 1 %); larger
// workgroups lose 3-10 %.  (All-zero buffers
// run up to 10 % faster than any other content on this memory system and must
// not be used for tuning.)
constexpr int kTableBlock = 64;
constexpr int kGatherUnroll = 2;
constexpr int kScatterUnroll = 2;
constexpr bool kTableNtLoad = true;
constexpr bool kTableNtStore = true;
constexpr long long kGatherTileElems = (long long)kTableBlock * kGatherUnroll * 8;
constexpr long long kScatterTileElems = (long long)kTableBlock * kScatterUnroll * 8;
// default grid cap in workgroups per compute unit.  Measured: one workgroup per
// tile (no cap reached) beats a persistent grid-stride grid by 5-10 % on every
// kernel of the path, so the cap is far above any tile count of interest.
constexpr int kFlatBlocksPerCu = 4096;
constexpr int kTableBlocksPerCu = 4096;
}  // namespace yafsdp
