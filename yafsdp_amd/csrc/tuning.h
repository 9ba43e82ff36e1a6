// Launch shapes of the shipped kernels (chosen by measurement on MI355X).
#pragma once
namespace yafsdp {
// flat kernels: workgroup size, units (8 elements) per lane per tile,
// non-temporal loads / stores
constexpr int kFlatBlock = 256;
constexpr int kFlatUnroll = 4;
constexpr bool kFlatNtLoad = true;
constexpr bool kFlatNtStore = true;
// gather-in / scatter-out: a tile is kTableBlock * kTableUnroll * 8 elements
constexpr int kTableBlock = 256;
constexpr int kTableUnroll = 4;
constexpr bool kTableNtLoad = true;
constexpr bool kTableNtStore = true;
constexpr long long kTableTileElems = (long long)kTableBlock * kTableUnroll * 8;
// default grid: workgroups per compute unit
constexpr int kFlatBlocksPerCu = 8;
constexpr int kTableBlocksPerCu = 8;
}  // namespace yafsdp
