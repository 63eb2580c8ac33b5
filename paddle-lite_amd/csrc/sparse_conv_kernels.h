// Launch interface of the gfx950 sparse 1x1 convolution kernels.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace pl {

// Output kinds of the kernels.
enum : int { kOutF32 = 0, kOutI8 = 1, kOutAcc32 = 2 };

struct DevAct {
  int type;  // lite_api::ActivationType value: 1 relu, 2 relu6, 4 leaky, 10 hard_swish
  float relu6_coef;
  float leaky_alpha;
  float hs_inv_scale;
  float hs_offset;
  float hs_threshold;
};

// One output row, or two rows that share an index list.
struct DevGroup {
  int row0;
  int nrows;
  uint32_t first;
  uint32_t count;
};

// Entries of an index list are taken this many at a time; every list is
// padded to a multiple of it with zero-weight entries.
#ifndef PL_WALK_BATCH
#define PL_WALK_BATCH 8
#endif
constexpr int kWalkBatch = PL_WALK_BATCH;

// Row-walk SpMM: arguments common to all instantiations.
struct WalkParams {
  const void* x;
  void* out;
  const DevGroup* groups;
  const uint32_t* kidx;  // per entry: input channel (fp32) or channel quad (int8)
  const uint32_t* wts;   // per entry: 1 or 2 dwords (float bits / 4 packed int8)
  const float* scale;    // int8 only
  const float* bias;     // may be null
  int n_groups;
  int groups_per_slice;
  int M, K;
  int kd;                // LDS tile rows: K (fp32, plus one all-zero row) or ceil(K/4) (int8)
  int hw;
  uint32_t P;            // batch * hw
  int vec;               // 1: hw % 4 == 0 and pointers 16-byte aligned
  DevAct act;
  int tiles, slices;     // filled in by the launcher
};

struct WalkConfig {
  bool int8;       // activations / weights are int8
  int out_kind;    // kOutF32 / kOutI8 / kOutAcc32
  int nrows;       // 1 unstructured, 2 semi
  int tile_pos;    // positions per workgroup tile: 16, 32, 64, 128 or 256
  int threads;     // 256, 512 or 1024
  int slices;      // grid.y
};

hipError_t LaunchRowWalk(const WalkConfig& cfg, const WalkParams& p, hipStream_t stream);

// fp32 row walk over channel chunks (chunk_walk_kernels.hip): a workgroup of
// kChunkWalkWaves wavefronts takes kChunkWalkTile positions and a slice of
// kChunkWalkWaves * groups_per_wave row groups (4 or 8; the half-precision
// walk always kChunkWalkGroups), and stages kChunkWalkChunk channels at a time.
constexpr int kChunkWalkTile = 256;
constexpr int kChunkWalkChunk = 64;
constexpr int kChunkWalkWaves = 8;
constexpr int kChunkWalkGroups = 8;

struct ChunkWalkParams {
  const void* x;
  void* out;
  const DevGroup* groups;  // row0 / nrows of every row group
  // [slice][chunk][wave][group of the wave]: first batch, number of entries
  const uint32_t* desc;
  const uint32_t* idx;     // per batch of four entries: four chunk-local channels, 8 bits each (kChunkWalkChunk = zero row)
  const uint32_t* wts;     // per batch: 4 entries x nrows float bit patterns
  const float* bias;       // may be null
  int n_groups;
  int n_chunks, slices;
  int groups_per_wave;     // 4 or 8, as the descriptors were built
  int M, K;
  int hw;
  uint32_t P;
  DevAct act;
  int tiles;               // filled in by the launcher
};

// Needs hw % 4 == 0 and 16-byte aligned x / out.
hipError_t LaunchChunkWalk(int nrows, const ChunkWalkParams& p, hipStream_t stream);

// fp32 walk with the whole tile and the index lists in LDS
// (tile_walk_kernels.hip): a workgroup of kTileWalkWaves wavefronts takes
// kTileWalkTile positions with all input channels; wavefront s walks the row
// groups of list stream s.
constexpr int kTileWalkTile = 128;
constexpr int kTileWalkRagged = 8;      // flag in TileWalkParams::pairs
// TileWalkParams::pairs without the flag: the form.  0: one row group per wavefront instruction, 1: two (tiles of
// 128 positions both), 2: four on tiles of 64 positions, 3: eight on tiles of 32, 4: sixteen on tiles of 16.
constexpr int kTileWalkForms = 5;
constexpr int TileWalkGroupsOf(int form) { return 1 << form; }
constexpr int TileWalkTileOf(int form) { return form <= 1 ? kTileWalkTile : 256 >> form; }  // for channel counts whose 128-position tile does not fit LDS (pairs only)
constexpr int kTileWalkWaves = 16;
constexpr int kTileWalkChunkBytes = 1536;  // piece of a list stream held in LDS per wavefront

struct TileWalkParams {
  const float* x;
  float* out;
  // List streams, kTileWalkChunkBytes at a time, as records of 16 + 16 * nrows
  // bytes.  A row group is a header record (first row | rows << 24, entries,
  // bias bit patterns of its rows) followed by one record per batch of four
  // entries: four byte offsets of channel rows in the tile (channel *
  // kTileWalkTile * 4; unused slots of the last batch point at the zero row
  // behind the last channel), then 4 x nrows float bit patterns (entry-major).
  // Records do not straddle chunks; every stream ends with one spare chunk.
  const void* stream;
  const uint32_t* stream_first;   // [kTileWalkWaves] first chunk of every stream; with `split`, [2 * kTileWalkWaves]: main part, spare part
  int K;
  int hw;
  uint32_t P;
  int tiles;                     // filled in by the launcher
  // 1: the row groups are dealt into a main and a spare part; the grid then has
  // split_slots workgroups per XCD (one per CU), more than any XCD has tiles.
  // 2: `parts` equal parts, as many workgroups per tile (parts x the tiles of
  // an XCD must not exceed split_slots); the stream tables then hold
  // parts x kTileWalkWaves entries.
  int16_t split;
  int8_t parts;
  // The form (above).  From 1 on the streams hold 2, 4, 8 or 16 row groups per step, padded to one length, their
  // records side by side: lanes [0, 64 / groups) walk the first group, the next 64 / groups lanes the second, ...,
  // four positions per lane; the byte offsets in the records are made for channel rows of the form's tile.
  // + kTileWalkRagged (not with form 0): hw is not a multiple of 4; tile and outputs are moved element by element
  int8_t pairs;
  // The first 56 bytes (kernarg_head.h) end behind act.type: what selects the tile, picks the activation and
  // addresses the first loads.
  DevAct act;
  const uint32_t* stream_groups;  // row groups in every stream, same shape as stream_first
  int n_groups;
  int M;
  int split_slots;
};

// LDS the kernel needs for K input channels.
size_t TileWalkLdsBytes(int K, int row_bytes = kTileWalkTile * 4);  // row_bytes: bytes per channel row of the tile
// Needs hw % 4 == 0 and 16-byte aligned x / out, or the ragged form.
hipError_t LaunchTileWalk(int nrows, const TileWalkParams& p, hipStream_t stream);

// Half-precision row walk (fp16_walk_kernels.hip).  Activation constants as
// binary16 bit patterns.
struct DevActH {
  int type;
  uint16_t alpha;         // relu6 bound or leaky slope
  uint16_t hs_offset;
  uint16_t hs_inv_scale;  // (half)(1.0 / scale)
  uint16_t hs_threshold;
};

// Half-precision walk over channel chunks (the layout of ChunkWalkParams; a
// weight entry is one dword, row 0 in the low half and row 1 in the high half).
struct HalfChunkWalkParams {
  const uint16_t* x;
  uint16_t* out;
  const DevGroup* groups;
  const uint32_t* desc;
  const uint32_t* idx;
  const uint32_t* wts;
  const uint16_t* bias;    // may be null
  int n_groups;
  int n_chunks, slices;
  int M, K;
  int hw;
  uint32_t P;
  DevActH act;
  int tiles;               // filled in by the launcher
};

// Needs hw % 4 == 0 and 8-byte aligned x / out.
hipError_t LaunchHalfChunkWalk(int nrows, const HalfChunkWalkParams& p, hipStream_t stream);

// Half-precision tile walk: the layout of TileWalkParams with pairs of row groups.  A tile holds 256 positions
// (the same 512 bytes per channel row, so the byte offsets in the list streams are those of the fp32 walk), a
// lane eight; or 128 positions (256 bytes per channel row, streams made for that), a lane four: twice the
// channels fit, and a map size that is a multiple of 4 is enough.  Weights and biases in the streams are binary16
// values doubled into a dword (value | value << 16).
constexpr int kHalfTileWalkTile = 256;
constexpr int kHalfTileWalkNarrowTile = 128;
// HalfTileWalkParams::form without the flag.  0 - 3: 2 / 4 / 8 / 16 row groups per wavefront instruction, eight
// positions per lane, on tiles of 256 / 128 / 64 / 32 positions (up to 271 / 543 / 1087 / 2175 channels); 4: the narrow
// form, pairs with four positions per lane on tiles of 128.
constexpr int kHalfTileWalkForms = 5;
constexpr int kHalfTileWalkNarrowForm = 4;
constexpr int HalfTileWalkGroupsOf(int form) { return form == kHalfTileWalkNarrowForm ? 2 : 2 << form; }
constexpr int HalfTileWalkTileOf(int form) { return form == kHalfTileWalkNarrowForm ? kHalfTileWalkNarrowTile : kHalfTileWalkTile >> form; }

struct HalfTileWalkParams {
  const uint16_t* x;
  uint16_t* out;
  const void* stream;
  const uint32_t* stream_first;
  int K;
  int hw;
  uint32_t P;
  int tiles;  // filled in by the launcher
  int16_t split;
  int8_t parts;
  int8_t form;  // the form (above); + kTileWalkRagged: the tile is staged and the outputs are stored value by value (any map size and alignment)
  // the first 56 bytes (kernarg_head.h) end behind act.type
  DevActH act;
  const uint32_t* stream_groups;
  int n_groups;
  int M;
  int split_slots;
};

// Eight positions per lane need hw % 8 == 0 and 16-byte aligned x / out, the narrow form hw % 4 == 0 and 8-byte
// alignment, the ragged flag lifts both; the streams must be made for the form's channel rows and groups per step.
hipError_t LaunchHalfTileWalk(int nrows, const HalfTileWalkParams& p, hipStream_t stream);

struct HalfWalkParams {
  const uint16_t* x;
  uint16_t* out;
  const DevGroup* groups;
  const uint32_t* kidx;   // per entry: input channel (K = the tile's zero row)
  const uint32_t* wts;    // per entry: weight of row 0 in the low half, of row 1 in the high half
  const uint16_t* bias;   // may be null
  int n_groups;
  int groups_per_slice;
  int M, K;
  int hw;
  uint32_t P;
  int pair;               // 1: hw even and x / out 4-byte aligned
  DevActH act;
  int tiles, slices;      // tiles filled in by the launcher
};

// tile_pos: 128, 64, 32 or 16 positions with (K + 1) * tile_pos * 2 bytes of LDS.
hipError_t LaunchHalfWalk(int nrows, int tile_pos, int threads, const HalfWalkParams& p, hipStream_t stream);

// Block MFMA SpMM (int8): dense 32x32 weight blocks pre-arranged in operand
// order, empty blocks skipped through a per-row-block bit mask.
struct MfmaParams {
  const int8_t* x;
  void* out;
  const void* wblocks;     // [row_blocks][ksteps][64 lanes][16 bytes]
  const uint32_t* kmask;   // [row_blocks][kmask_words] bit ks set = block (rb, ks) has a nonzero
  int kmask_words;         // ceil(ksteps / 32)
  const float* scale;      // padded to 32 * row_blocks
  const float* bias;       // padded likewise (zeros when the op has no bias)
  int row_blocks;
  int ksteps;              // ceil(K / 32)
  int M, K;
  int hw;
  uint32_t P;              // batch * hw
  int small;               // 1: input and output tensors are each below 2 GB
  DevAct act;
  // filled in by the launcher
  int vec;                 // hw >= 4: positions are handled four at a time by dword access
  int quad_aligned;        // hw % 4 == 0: every quad is complete
  int qpi;                 // quads per image = ceil(hw / 4)
  uint32_t total_quads;    // batch * qpi
  int tiles;               // tiles of tile_quads quads
  int tile_quads;
  int sub_tiles;           // tiles per workgroup (1, 2 or 4)
  int row_groups;          // groups of four row blocks
  int i8_stage;            // int8 output is regrouped through LDS for 16-byte stores
  // streaming variant (tiles cut per image, workgroups walk over tiles)
  int stream_tpi;          // tiles per image
  int stream_tiles;        // batch * stream_tpi
  int stream_lanes;        // workgroups per XCD and row group = tile stride of a workgroup
};

struct MfmaConfig {
  int out_kind;
  int ks_max;          // 2, 4, 8, 16 or 32 (>= ksteps)
  int tile_quads;      // 1..32 position quads per workgroup tile
  int sub_tiles;       // several tiles per workgroup for at most 64 input channels: 0 never, 1 when enough workgroups remain, 2 always
  int i8_wide_stores;  // int8 output: regroup through LDS into 16-byte stores
  int stream;          // streaming variant for large maps with 128 / 256 channels: 0 never, 1 when the shape suits it, 2 whenever the shape allows
  int cus;             // compute units of the device
};

hipError_t LaunchBlockMfma(const MfmaConfig& cfg, const MfmaParams& p, hipStream_t stream);

// Image MFMA SpMM (int8, image_mfma_kernels.hip): one workgroup per (image,
// 128 output rows) with the whole image's activations in LDS.
struct ImageMfmaParams {
  // the first 56 bytes: what the first loads of a kernel need (kernarg_head.h)
  const int8_t* x;
  void* out;
  // dense 16x64 weight tiles in matrix-core operand order:
  // [row group of 128][class rho = 0..3][tile j = 0..1][k-step][64 lanes][16 bytes];
  // lane l of tile (rho, j) holds row rho + 4 (16 j + l % 16), channels 64 ks + 16 (l / 16) .. + 15
  const void* wtiles;
  int K;
  int hw;              // positions a work item takes: the whole map (H * W), or one slab of it (image_rows_kernels.hip)
  // filled in by the launcher
  int pitch;           // positions of the whole map = bytes between the channel rows of x and elements between output rows
  int slabs;           // slabs per image (1: the whole map is one item)
  int items, per_xcd;  // work items (image, slab, row group) in all and per XCD
  int row_groups;      // M / 128
  int batch;
  // behind the head
  int M;
  int qpi;             // position quads per item = hw / 4
  const float* scale;  // output-row order, at least M entries
  const float* bias;   // likewise (zeros when the op has no bias)
  DevAct act;
  // filled in by the launcher
  int kgs;             // 16-byte cells per channel group in LDS (a multiple of 16)
  int dma_full, dma_rem_lanes;  // 1 KB pieces of a channel group and the lanes of the last, partial piece
  int align;           // fp32 / int32 output: windows shifted onto 64-byte sector boundaries
  // set by the caller of LaunchImageMfma: wtiles holds the tiles in the channel order of the regrouping by
  // transposing LDS reads (byte b of lane group g of k-step ks = channel 64 ks + 4 (8 (g % 2) + b % 8) + 2 (b / 8) + g / 2);
  // only where ImageMfmaRegroupsByTransposingReads(K, hw)
  int tr_regroup;
};

// M a multiple of 128, K = 128, 256 or 512, hw a multiple of 4 in [16, 256]
// and the image's cells within the LDS of a CU; or 7 x 7 maps (hw = 49) with
// K = 256, 512 or 1024 (two images per workgroup).
bool ImageMfmaFits(int M, int K, int hw);
bool ImageMfmaRegroupsByTransposingReads(int K, int hw);
// Needs ImageMfmaFits and 16-byte aligned x / out.
hipError_t LaunchImageMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream);

// The same work item with the image kept in LDS as it lies in memory and the
// operands read with transposing LDS reads (image_tr_kernels.hip).  wtiles
// then holds the tiles in that kernel's channel order:
// [row group][rho][j][step = 2 (c / 128) + c % 2][64 lanes][16 bytes], lane l
// byte b of a step holding row rho + 4 (16 j + l % 16) and channel
// 128 (step / 2) + step % 2 + 64 (b / 8) + 4 (8 (g % 2) + b % 8) + 2 (g / 2), g = l / 16.
// M a multiple of 128, K = 128, 256 or 512, hw = 4 (mod 8) from 20 on and
// the image plus 41 KB of staging buffers within the LDS of a CU.
// The image kernel with one row tile (rows 8 apart) per wavefront and the image brought in through registers
// (image_rows_kernels.hip): wtiles = [row group][tile w = 0 .. 7][k-step][64 lanes][16 bytes], lane l of tile w
// holds row w + 8 (l % 16), channels 64 ks + 16 (l / 16) .. + 15.  M a multiple of 128, K = 128, 256 or 512, hw a
// multiple of 4 in [16, 256] and the image's cells within the LDS of a CU; x 4-byte and out 16-byte aligned.
bool ImageRowsMfmaFits(int M, int K, int hw);
// Larger maps of a multiple of 196 positions (28 x 28, 56 x 56, 112 x 112): the same kernel on slabs of 196
// positions, one work item per (image, slab, 128 output rows).
bool ImageRowsSlabFits(int M, int K, int hw);
hipError_t LaunchImageRowsMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream);

bool ImageTrMfmaFits(int M, int K, int hw);
// Needs ImageTrMfmaFits and 16-byte aligned x / out.
hipError_t LaunchImageTrMfma(int out_kind, const ImageMfmaParams& p, hipStream_t stream);

// Largest dynamic LDS size a kernel of this library may be given.
constexpr int kMaxLdsBytes = 160 * 1024;
constexpr int kMfmaTilePos = 128;
// More than 32 k-steps (1024 input channels): the block MFMA kernel takes
// them this many at a time through one LDS tile.
constexpr int kLoopChunk = 8;

// Precision changes around an int8 convolution (calib_kernels.hip).
hipError_t LaunchFp32ToInt8(const float* x, int8_t* out, int64_t n, float scale, hipStream_t stream);
hipError_t LaunchInt8ToFp32(const int8_t* x, float* out, int64_t n, float scale, hipStream_t stream);

}  // namespace pl
