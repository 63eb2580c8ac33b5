// C ABI of the gfx950 sparse 1x1 convolution: layout validation, one-time
// conversion of the compressed weights into the device-side forms, launch
// selection.  No CPU compute path exists here: without a device
// pl_sparse_conv_prepare() fails with PL_ERR_NO_DEVICE.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdarg>
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cmath>
#include <cstring>
#include <initializer_list>
#include <memory>
#include <new>
#include <string>
#include <utility>
#include <vector>

#include "../../include/pl_sparse_conv.h"
#include "dwconv_kernels.h"
#include "sparse_conv_kernels.h"
#include "sparse_layout.h"

namespace {

thread_local std::string g_last_error;

int Fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_last_error = buf;
  return code;
}

int FailHip(hipError_t e, const char* what) {
  return Fail(PL_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

// Owning device allocation.
struct DevBuf {
  void* ptr = nullptr;
  size_t bytes = 0;
  DevBuf() = default;
  DevBuf(const DevBuf&) = delete;
  DevBuf& operator=(const DevBuf&) = delete;
  ~DevBuf() { Reset(); }
  void Reset() {
    if (ptr) (void)hipFree(ptr);
    ptr = nullptr;
    bytes = 0;
  }
  hipError_t Upload(const void* host, size_t n) {
    Reset();
    if (n == 0) n = 16;  // keep kernels' pointer arguments valid
    hipError_t e = hipMalloc(&ptr, n);
    if (e != hipSuccess) {
      ptr = nullptr;
      return e;
    }
    bytes = n;
    if (host) e = hipMemcpy(ptr, host, n, hipMemcpyHostToDevice);
    return e;
  }
};

pl::DevAct ToDevAct(const pl_activation& a) {
  pl::DevAct d{};
  d.type = a.type;
  d.relu6_coef = a.relu6_coef;
  d.leaky_alpha = a.leaky_alpha;
  // the math functions form 1.0 / scale in double and narrow it
  // (lite/backends/arm/math/sparse_conv_impl.cc:1211)
  d.hs_inv_scale = a.type == PL_ACT_HARD_SWISH ? static_cast<float>(1.0 / a.hs_scale) : 0.0f;
  d.hs_offset = a.hs_offset;
  d.hs_threshold = a.hs_threshold;
  return d;
}

int CeilDiv(int a, int b) { return (a + b - 1) / b; }

// double (or float, which widens exactly) -> IEEE binary16 bit pattern with
// one rounding to nearest even (what the reference's fp32_to_fp16 and
// static_cast<float16_t> do).
uint16_t HalfBits(double f) {
  uint64_t u;
  std::memcpy(&u, &f, 8);
  const uint16_t sign = static_cast<uint16_t>((u >> 48) & 0x8000u);
  const uint64_t a = u & 0x7fffffffffffffffull;
  if (a > 0x7ff0000000000000ull) return static_cast<uint16_t>(sign | 0x7e00u);  // NaN
  const double mag = std::fabs(f);
  if (mag >= 65520.0) return static_cast<uint16_t>(sign | 0x7c00u);  // rounds to infinity
  if (mag < 2.9802322387695312e-08) return sign;                     // < 2^-25 rounds to zero
  const int e = static_cast<int>(a >> 52) - 1023;                    // unbiased (mag is a normal double here)
  const uint64_t m = (a & 0xfffffffffffffull) | 0x10000000000000ull;  // 53-bit significand
  // keep 10 fraction bits (fewer for subnormal results)
  const int shift = e >= -14 ? 42 : 42 + (-14 - e);
  const uint64_t kept = m >> shift, rest = m & ((1ull << shift) - 1ull), half = 1ull << (shift - 1);
  const uint32_t r = static_cast<uint32_t>(kept + ((rest > half || (rest == half && (kept & 1ull))) ? 1ull : 0ull));
  if (e >= -14) {
    // r carries the implicit bit at position 10: adding it to the exponent
    // field below also handles the carry out of the fraction
    return static_cast<uint16_t>(sign | ((static_cast<uint32_t>(e + 14) << 10) + r));
  }
  return static_cast<uint16_t>(sign | r);  // subnormal; r == 1024 is the smallest normal number
}

pl::DevActH ToDevActH(const pl_activation& a) {
  pl::DevActH d{};
  d.type = a.type;
  if (a.type == PL_ACT_RELU6) d.alpha = HalfBits(a.relu6_coef);
  if (a.type == PL_ACT_LEAKY_RELU) d.alpha = HalfBits(a.leaky_alpha);
  if (a.type == PL_ACT_HARD_SWISH) {
    // (float16_t)(1.0 / scale): formed in double and narrowed once
    // (lite/backends/arm/math/fp16/sparse_conv_fp16.cc:1318-1322)
    d.hs_offset = HalfBits(a.hs_offset);
    d.hs_inv_scale = HalfBits(1.0 / static_cast<double>(a.hs_scale));
    d.hs_threshold = HalfBits(a.hs_threshold);
  }
  return d;
}

}  // namespace

// List streams of a tile walk (fp32, or half precision with a given number of bytes per channel row of the tile).
struct TileWalkStreams {
  DevBuf stream, first, desc;
  int built = 0;  // uploaded
  int row_bytes = 0;  // bytes per channel row of the LDS tile the byte offsets in the records are made for
  int groups = 1;     // row groups per step of a stream (records side by side)
  int form = 0;       // fp32: TileWalkParams::pairs without flags
  // host copy of the streams and, per header record, (word index of its bias, first row | rows << 24):
  // the headers carry the bias, so a new bias is patched in here and the streams are uploaded again
  std::vector<uint32_t> host_stream;
  std::vector<std::pair<uint32_t, uint32_t>> bias_slots;
  int64_t stream_work = 0;  // work units (entry batches + 2 per row group) of the fullest of the sixteen unsplit streams
  size_t DeviceBytes() const { return stream.bytes + first.bytes + desc.bytes; }
};

struct pl_sparse_conv_handle {
  int device = 0;
  int kind = PL_KIND_FP32;
  int algo = PL_ALGO_ROW_WALK;
  int oc = 0, ic = 0;
  bool int8 = false;
  bool semi = false;
  bool has_bias = false;
  pl::DevAct act{};
  int64_t nnz = 0, stored = 0, entries = 0;
  // row walk
  int n_groups = 0;
  int kd = 0;
  int64_t walk_entries = 0;
  DevBuf groups, kidx, wts;
  // fp32 row walk over channel chunks (built beside the plain form)
  DevBuf cw_desc, cw_idx, cw_wts;
  int cw_chunks = 0, cw_slices = 0;
  // tile walk (whole tile and lists in LDS).  tw: fp32 in the form with the largest tile that holds all channels
  // (128 positions, or 64 / 32 / 16 with 4 / 8 / 16 row groups per step); half precision with 256 positions per
  // tile.  tw_narrow: half precision with 128 positions per tile (256-byte channel rows), for more channels and for
  // maps whose size is a multiple of 4 but not of 8.
  TileWalkStreams tw, tw_narrow;
  int walk_split = -1;          // sixteenths of the row groups' work dealt to the CUs without a tile: -1 by rule, 0 never, 1 .. 8 forced
  int walk_tiled = 1;            // 0 never, 1 when the problem suits it, 2 whenever the shape allows
  bool walk_pairs = true;        // the tile walk's streams hold pairs of row groups (two per wavefront instruction)
  int cw_groups = 8;  // row groups per wavefront of the fp32 walk over channel chunks: 8, or 4 on request
  int walk_chunked = 1;  // 0 never, 1 when the problem is large enough, 2 whenever the shape allows
  bool walk_plain_fits = true;  // false: more channels than the plain walk's LDS tile holds, only the chunked walk can run
  // half-precision row walk
  bool half = false;
  pl::DevActH act_h{};
  DevBuf hw_kidx, hw_wts, hw_bias;
  // block MFMA
  int row_blocks = 0, ksteps = 0, kmask_words = 1;
  int64_t blocks_present = 0;
  DevBuf wblocks, kmask;
  int wg_slots = 512;       // workgroups resident at once (2 per CU)
  int wg_slots_default = 512;  // the same before any override: twice the device's CU count
  int mfma_stream = 1;      // streaming block MFMA: 0 never, 1 when the shape suits it, 2 whenever the shape allows
  int mfma_i8_wide = 1;
  int mfma_tile_quads = 0;  // 0 = chosen per problem
  int mfma_sub_tiles = 1;   // several tiles per workgroup for <= 64 input channels: 0 never, 1 when enough workgroups remain, 2 always
  // image MFMA (dense 16x64 tiles, rows of a tile four apart)
  DevBuf wtiles;
  DevBuf wtiles_rg;      // the same tiles in the channel order of the regrouping by transposing LDS reads (ic = 512)
  bool image_tr_regroup = true;
  DevBuf wtiles_tr;      // the same tiles in the channel order of the kernel with transposing LDS reads
  DevBuf wtiles_rows;    // tiles of rows 8 apart, for the image kernel with one row tile per wavefront
  int image_kernel = 0;  // 0 by rule, 1 regrouping kernel, 2 transposing-read kernel
  // int8 handles prepared with PL_ALGO_AUTO hold several forms and choose per call
  bool auto_int8 = false;
  int image_min_items = 1;  // fewest (image, 128-row group) work items for which the image kernel is chosen
  bool auto_walk = false;   // an automatic int8 handle that also holds the row walk's lists
  // row-walk tuning read once at prepare (0 = chosen per problem)
  int walk_tile = 0, walk_threads = 0, walk_slices = 0;
  // epilogue
  DevBuf scale, bias;
  int padded_rows = 0;

  int64_t DeviceBytes() const {
    return static_cast<int64_t>(groups.bytes + kidx.bytes + wts.bytes + cw_desc.bytes + cw_idx.bytes + cw_wts.bytes + hw_kidx.bytes + hw_wts.bytes + hw_bias.bytes + wblocks.bytes + kmask.bytes + wtiles.bytes + wtiles_rg.bytes + wtiles_tr.bytes + wtiles_rows.bytes + tw.DeviceBytes() + tw_narrow.DeviceBytes() + scale.bytes + bias.bytes);
  }
};

namespace {

int OutKind(int kind) {
  switch (kind) {
    case PL_KIND_INT8_INT8:
      return pl::kOutI8;
    case PL_KIND_INT8_ACC32:
      return pl::kOutAcc32;
    default:
      return pl::kOutF32;
  }
}

// Device-side form for the row walk: per group an index list; int8 weights
// of one channel quad are merged into one dword so that one v_dot4 consumes
// them.
int BuildRowWalk(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int nr = L.semi ? 2 : 1;
  std::vector<pl::DevGroup> groups;
  std::vector<uint32_t> kidx, wts;
  groups.reserve(L.groups.size());
  for (const pl::RowGroup& g : L.groups) {
    pl::DevGroup d;
    d.row0 = g.row0;
    d.nrows = g.nrows;
    d.first = static_cast<uint32_t>(kidx.size());
    if (!h->int8) {
      for (uint32_t j = 0; j < g.count; ++j) {
        kidx.push_back(L.ic_index[g.first + j]);
        wts.push_back(L.w0[g.first + j]);
        if (nr == 2) wts.push_back(L.w1[g.first + j]);
      }
    } else {
      uint32_t j = 0;
      while (j < g.count) {
        const uint32_t q = L.ic_index[g.first + j] >> 2;
        uint32_t p0 = 0, p1 = 0;
        while (j < g.count && (L.ic_index[g.first + j] >> 2) == q) {
          const int sh = 8 * (L.ic_index[g.first + j] & 3u);
          p0 |= (L.w0[g.first + j] & 0xffu) << sh;
          p1 |= (L.w1[g.first + j] & 0xffu) << sh;
          ++j;
        }
        kidx.push_back(q);
        wts.push_back(p0);
        if (nr == 2) wts.push_back(p1);
      }
    }
    // The kernel takes entries kWalkBatch at a time.  Padding entries have
    // zero weights; fp32 ones read the all-zero row that the kernel appends
    // to its tile (index ic), so that a non-finite input cannot leak in.
    while ((kidx.size() - d.first) % pl::kWalkBatch != 0) {
      kidx.push_back(h->int8 ? 0u : static_cast<uint32_t>(L.ic));
      wts.push_back(0u);
      if (nr == 2) wts.push_back(0u);
    }
    d.count = static_cast<uint32_t>(kidx.size()) - d.first;
    groups.push_back(d);
  }
  h->n_groups = static_cast<int>(groups.size());
  h->kd = h->int8 ? CeilDiv(L.ic, 4) : L.ic;
  h->walk_entries = static_cast<int64_t>(kidx.size());
  hipError_t e = h->groups.Upload(groups.data(), groups.size() * sizeof(pl::DevGroup));
  if (e == hipSuccess) e = h->kidx.Upload(kidx.data(), kidx.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = h->wts.Upload(wts.data(), wts.size() * sizeof(uint32_t));
  if (e != hipSuccess) return FailHip(e, "uploading the row-walk index");
  return PL_OK;
}

// Device-side form for the half-precision walk: groups as for the plain walk,
// per entry the channel and the weights of both rows as binary16 in one
// dword; lists padded to kWalkBatch with zero-weight entries that read the
// tile's zero row (index ic).
int BuildHalfWalk(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  std::vector<pl::DevGroup> groups;
  std::vector<uint32_t> kidx, wts;
  for (const pl::RowGroup& g : L.groups) {
    pl::DevGroup d;
    d.row0 = g.row0;
    d.nrows = g.nrows;
    d.first = static_cast<uint32_t>(kidx.size());
    for (uint32_t j = 0; j < g.count; ++j) {
      float w0, w1 = 0.f;
      std::memcpy(&w0, &L.w0[g.first + j], 4);
      if (g.nrows == 2) std::memcpy(&w1, &L.w1[g.first + j], 4);
      kidx.push_back(L.ic_index[g.first + j]);
      wts.push_back(static_cast<uint32_t>(HalfBits(w0)) | (static_cast<uint32_t>(HalfBits(w1)) << 16));
    }
    while ((kidx.size() - d.first) % pl::kWalkBatch != 0) {
      kidx.push_back(static_cast<uint32_t>(L.ic));
      wts.push_back(0u);
    }
    d.count = static_cast<uint32_t>(kidx.size()) - d.first;
    groups.push_back(d);
  }
  h->n_groups = static_cast<int>(groups.size());
  hipError_t e = h->groups.Upload(groups.data(), groups.size() * sizeof(pl::DevGroup));
  if (e == hipSuccess) e = h->hw_kidx.Upload(kidx.empty() ? nullptr : kidx.data(), kidx.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = h->hw_wts.Upload(wts.empty() ? nullptr : wts.data(), wts.size() * sizeof(uint32_t));
  if (e != hipSuccess) return FailHip(e, "uploading the half-precision index");
  return PL_OK;
}

int UploadHalfBias(pl_sparse_conv_handle* h, const float* bias) {
  if (!bias) return PL_OK;
  std::vector<uint16_t> b(static_cast<size_t>(h->oc));
  for (int i = 0; i < h->oc; ++i) b[i] = HalfBits(bias[i]);
  const hipError_t e = h->hw_bias.Upload(b.data(), b.size() * sizeof(uint16_t));
  if (e != hipSuccess) return FailHip(e, "uploading biases");
  h->has_bias = true;
  return PL_OK;
}

// Device-side form for the fp32 walk over channel chunks: per (slice, chunk,
// wavefront, group of the wavefront) the batches of four entries whose channel
// lies in the chunk, in index order, padded with zero-weight entries that
// point at the tile's zero row.
// half: one weight dword per entry, the two rows' binary16 patterns in its halves
// fp32: the descriptor counts entries (the last batch of a list is walked up
// to its last real entry) and a wavefront owns h->cw_groups row groups; half:
// it counts batches and a wavefront owns kChunkWalkGroups.
int BuildChunkWalk(const pl::DecodedLayout& L, pl_sparse_conv_handle* h, bool half = false) {
  const int nr = L.semi ? 2 : 1;
  const int groups_per_wave = half ? pl::kChunkWalkGroups : h->cw_groups;
  const int per_slice = pl::kChunkWalkWaves * groups_per_wave;
  const int n_groups = static_cast<int>(L.groups.size());
  const int slices = CeilDiv(n_groups, per_slice);
  const int chunks = CeilDiv(L.ic, pl::kChunkWalkChunk);
  std::vector<uint32_t> desc(static_cast<size_t>(slices) * chunks * per_slice * 2, 0u);
  std::vector<uint32_t> idx, wts;
  for (int sl = 0; sl < slices; ++sl) {
    for (int c = 0; c < chunks; ++c) {
      for (int gl = 0; gl < per_slice; ++gl) {  // gl = wave * groups-per-wave + group of the wave
        const int g = sl * per_slice + gl;
        uint32_t* d = &desc[((static_cast<size_t>(sl) * chunks + c) * per_slice + gl) * 2];
        d[0] = static_cast<uint32_t>(idx.size());
        if (g >= n_groups) continue;
        const pl::RowGroup& rg = L.groups[g];
        uint32_t packed = 0, entries = 0;
        int fill = 0;
        auto flush = [&]() {
          for (; fill < 4; ++fill) {  // padding entries: zero row, zero weights
            packed |= static_cast<uint32_t>(pl::kChunkWalkChunk) << (8 * fill);
            for (int r = 0; r < (half ? 1 : nr); ++r) wts.push_back(0u);
          }
          idx.push_back(packed);
          packed = 0;
          fill = 0;
        };
        for (uint32_t j = 0; j < rg.count; ++j) {
          const uint32_t k = L.ic_index[rg.first + j];
          if (static_cast<int>(k / pl::kChunkWalkChunk) != c) continue;
          ++entries;
          packed |= (k % pl::kChunkWalkChunk) << (8 * fill);
          if (half) {
            float w0, w1 = 0.f;
            std::memcpy(&w0, &L.w0[rg.first + j], 4);
            if (nr == 2) std::memcpy(&w1, &L.w1[rg.first + j], 4);
            wts.push_back(static_cast<uint32_t>(HalfBits(w0)) | (static_cast<uint32_t>(HalfBits(w1)) << 16));
          } else {
            wts.push_back(L.w0[rg.first + j]);
            if (nr == 2) wts.push_back(L.w1[rg.first + j]);
          }
          if (++fill == 4) flush();
        }
        if (fill > 0) flush();
        d[1] = half ? static_cast<uint32_t>(idx.size()) - d[0] : entries;
      }
    }
  }
  h->cw_chunks = chunks;
  h->cw_slices = slices;
  hipError_t e = h->cw_desc.Upload(desc.data(), desc.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = h->cw_idx.Upload(idx.empty() ? nullptr : idx.data(), idx.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = h->cw_wts.Upload(wts.empty() ? nullptr : wts.data(), wts.size() * sizeof(uint32_t));
  if (e != hipSuccess) return FailHip(e, "uploading the chunked row-walk index");
  return PL_OK;
}

// Device-side form for the tile walks (fp32 and half precision): the row groups are dealt to
// kTileWalkWaves list streams (longest list first, each to the stream with the
// least work so far); a stream is the concatenation of its groups' batches of
// four entries as records of byte offsets and weights.  In half precision a weight or bias word is the
// binary16 value doubled (value | value << 16) and the streams always hold pairs.
// Main / spare divisions of the tile walk's row groups that are prepared: spare shares of 1/16 .. 8/16.
constexpr int kTileWalkSplits = 8;
// Equal divisions that are prepared (two equal parts are the 8/16 division above).
constexpr int kTileWalkEqualParts[] = {3, 4, 5, 6, 8, 10};

uint32_t DoubledHalf(uint32_t float_bits) {
  float v;
  std::memcpy(&v, &float_bits, 4);
  const uint32_t b = HalfBits(v);
  return b | (b << 16);
}

int BuildTileWalk(const pl::DecodedLayout& L, const float* bias, pl_sparse_conv_handle* h, TileWalkStreams* tw, bool half, int row_bytes, int groups_per_step) {
  tw->built = 0;
  tw->row_bytes = row_bytes;
  tw->groups = groups_per_step;
  if (pl::TileWalkLdsBytes(L.ic, row_bytes) > static_cast<size_t>(pl::kMaxLdsBytes)) return PL_OK;  // too many channels for one tile: other walks
  const int nr = L.semi ? 2 : 1;
  const int streams = pl::kTileWalkWaves;
  const int n_groups = static_cast<int>(L.groups.size());
  std::vector<int> order(n_groups);
  for (int g = 0; g < n_groups; ++g) order[g] = g;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return L.groups[a].count > L.groups[b].count; });
  // A unit is what one wavefront instruction walks: one row group, or G of about the same length - neighbours
  // in the order by length - of which the shorter ones are padded with entries of weight zero that point at the
  // tile's zero row; a last unit without enough groups gets empty ones (no rows).
  constexpr int kMaxG = 16;
  const int G = groups_per_step;
  if (G < 1 || G > kMaxG) return Fail(PL_ERR_BAD_ARG, "bad number of row groups per step");
  auto word = [&](uint32_t float_bits) { return half ? DoubledHalf(float_bits) : float_bits; };
  struct Unit {
    int g[kMaxG];    // row groups (-1: none)
    uint32_t count;  // entries walked
  };
  std::vector<Unit> units;
  for (int i = 0; i < n_groups; i += G) {
    Unit un;
    for (int k = 0; k < kMaxG; ++k) un.g[k] = k < G && i + k < n_groups ? order[i + k] : -1;
    un.count = L.groups[un.g[0]].count;  // sorted: the first is the longest
    units.push_back(un);
  }
  const int n_units = static_cast<int>(units.size());
  std::vector<int> unit_order(n_units);
  for (int u = 0; u < n_units; ++u) unit_order[u] = u;
  auto work = [&](int u) { return static_cast<int64_t>((units[u].count + 3) / 4 + 2); };  // batches, plus the unit's epilogue
  const uint32_t rec_words = 4 + 4 * nr;
  const uint32_t unit_words = static_cast<uint32_t>(G) * rec_words;  // the records of a step side by side
  const uint32_t chunk_words = pl::kTileWalkChunkBytes / 4;
  const uint32_t recs_per_chunk = chunk_words / unit_words;
  const uint32_t zero_row = static_cast<uint32_t>(L.ic) * static_cast<uint32_t>(row_bytes);
  std::vector<uint32_t>& stream = tw->host_stream;
  stream.clear();
  tw->bias_slots.clear();
  std::vector<uint32_t> first, counts;
  // Streams for the given units (largest first): each unit goes to the stream with the least work so far.
  // Sixteen streams make one part.  Returns the work of the fullest stream.
  auto emit = [&](const std::vector<int>& part, int n_streams) {
    std::vector<std::vector<int>> members(n_streams);
    std::vector<int64_t> load(n_streams, 0);
    for (int u : part) {
      int best = 0;
      for (int s2 = 1; s2 < n_streams; ++s2)
        if (load[s2] < load[best]) best = s2;
      members[best].push_back(u);
      load[best] += work(u);
    }
    for (int s2 = 0; s2 < n_streams; ++s2) {
      first.push_back(static_cast<uint32_t>(stream.size() / chunk_words));
      counts.push_back(static_cast<uint32_t>(members[s2].size()));
      uint32_t recs = 0;
      auto pad_chunk = [&]() {
        while (stream.size() % chunk_words != 0) stream.push_back(0u);
      };
      auto put = [&](const uint32_t* rec) {
        if (recs == recs_per_chunk) {  // records do not straddle chunks
          pad_chunk();
          recs = 0;
        }
        stream.insert(stream.end(), rec, rec + unit_words);
        ++recs;
      };
      for (int u : members[s2]) {
        const Unit& un = units[u];
        uint32_t rec[kMaxG * 12] = {0};
        const int* side_groups = un.g;
        const int sides = G;
        for (int side = 0; side < sides; ++side) {
          uint32_t* r = rec + side * rec_words;
          r[1] = un.count;
          if (side_groups[side] < 0) continue;  // no partner: no rows
          const pl::RowGroup& rg = L.groups[side_groups[side]];
          r[0] = static_cast<uint32_t>(rg.row0) | (static_cast<uint32_t>(rg.nrows) << 24);
          if (bias) {
            uint32_t b0 = 0, b1 = 0;
            std::memcpy(&b0, &bias[rg.row0], 4);
            if (rg.nrows == 2) std::memcpy(&b1, &bias[rg.row0 + 1], 4);
            r[2] = word(b0);
            if (rg.nrows == 2) r[3] = word(b1);
          }
        }
        put(rec);
        for (int side = 0; side < sides; ++side)
          if (side_groups[side] >= 0) tw->bias_slots.emplace_back(static_cast<uint32_t>(stream.size() - unit_words + side * rec_words + 2), rec[side * rec_words]);
        for (uint32_t e0 = 0; e0 < un.count; e0 += 4) {
          for (int side = 0; side < sides; ++side) {
            uint32_t* r = rec + side * rec_words;
            const pl::RowGroup* rg = side_groups[side] >= 0 ? &L.groups[side_groups[side]] : nullptr;
            for (uint32_t e = 0; e < 4; ++e) {
              const bool real = rg != nullptr && e0 + e < rg->count;
              r[e] = real ? L.ic_index[rg->first + e0 + e] * static_cast<uint32_t>(row_bytes) : zero_row;
              r[4 + e * nr] = real ? word(L.w0[rg->first + e0 + e]) : 0u;
              if (nr == 2) r[4 + e * nr + 1] = real ? word(L.w1[rg->first + e0 + e]) : 0u;
            }
          }
          put(rec);
        }
      }
      pad_chunk();
      stream.insert(stream.end(), chunk_words, 0u);  // the spare chunk the prefetch may touch
    }
    return *std::max_element(load.begin(), load.end());
  };
  // Set 0: all units in one part.  Sets 1 .. kTileWalkSplits: a spare part with about s / 16 of the work
  // (a mix of sizes: going through the units from the largest, a unit joins the spare part whenever that
  // keeps the part at or below its share), the rest in the main part.
  tw->stream_work = emit(unit_order, streams);
  for (int s16 = 1; s16 <= kTileWalkSplits; ++s16) {
    std::vector<int> main_part, spare_part;
    int64_t all_w = 0, spare_w = 0;
    for (int u : unit_order) {
      const int64_t w = work(u);
      all_w += w;
      if ((spare_w + w) * 16 <= static_cast<int64_t>(s16) * all_w) {
        spare_part.push_back(u);
        spare_w += w;
      } else {
        main_part.push_back(u);
      }
    }
    emit(main_part, streams);
    emit(spare_part, streams);
  }
  // Equal parts for problems with at most half as many tiles as CUs: n workgroups per tile, each with a
  // sixteenth-of-n share of the units.
  for (int n : kTileWalkEqualParts) emit(unit_order, streams * n);
  hipError_t e = tw->stream.Upload(stream.data(), stream.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = tw->first.Upload(first.data(), first.size() * sizeof(uint32_t));
  if (e == hipSuccess) e = tw->desc.Upload(counts.data(), counts.size() * sizeof(uint32_t));
  if (e != hipSuccess) return FailHip(e, "uploading the tile-walk list streams");
  tw->built = 1;
  return PL_OK;
}

// Device-side form for the block MFMA path: the weight matrix as dense
// 32x32 int8 blocks in matrix-core operand order, plus the mask of blocks
// that hold a nonzero.
int BuildBlockMfma(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int rbs = CeilDiv(L.oc, 32), kss = CeilDiv(L.ic, 32);
  std::vector<int8_t> blocks(static_cast<size_t>(rbs) * kss * 64 * 16, 0);
  const int words = CeilDiv(kss, 32);  // mask words per row block
  std::vector<uint32_t> mask(static_cast<size_t>(rbs) * words, 0u);
  auto put = [&](int row, uint32_t c, uint32_t wbits) {
    const int8_t w = static_cast<int8_t>(wbits & 0xffu);
    if (w == 0) return;
    const int rb = row >> 5, i = row & 31;
    const int ks = c >> 5, kk = c & 31;
    const int lane = i + 32 * (kk >> 4), t = kk & 15;
    blocks[((static_cast<size_t>(rb) * kss + ks) * 64 + lane) * 16 + t] = w;
    mask[static_cast<size_t>(rb) * words + (ks >> 5)] |= 1u << (ks & 31);
  };
  for (const pl::RowGroup& g : L.groups) {
    for (uint32_t j = 0; j < g.count; ++j) {
      put(g.row0, L.ic_index[g.first + j], L.w0[g.first + j]);
      if (g.nrows == 2) put(g.row0 + 1, L.ic_index[g.first + j], L.w1[g.first + j]);
    }
  }
  h->row_blocks = rbs;
  h->ksteps = kss;
  h->kmask_words = words;
  h->blocks_present = 0;
  for (uint32_t m : mask) h->blocks_present += __builtin_popcount(m);
  hipError_t e = h->wblocks.Upload(blocks.data(), blocks.size());
  if (e == hipSuccess) e = h->kmask.Upload(mask.data(), mask.size() * sizeof(uint32_t));
  if (e != hipSuccess) return FailHip(e, "uploading the weight blocks");
  return PL_OK;
}

// Device-side form for the image MFMA path: the weight matrix as dense 16x64
// int8 tiles in matrix-core operand order.  The 16 rows of a tile are four
// apart (rho, rho + 4, ...): they all start at the same offset inside a
// 64-byte sector of an fp32 output whose rows are H*W floats long.
int BuildImageMfma(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int kss = L.ic / 64;
  std::vector<int8_t> tiles(static_cast<size_t>(L.oc) * L.ic, 0);
  auto put = [&](int row, uint32_t c, uint32_t wbits) {
    const int8_t w = static_cast<int8_t>(wbits & 0xffu);
    if (w == 0) return;
    const int rg = row / 128, rl = row % 128;
    const int rho = rl & 3, m32 = rl >> 2;  // row = rg * 128 + rho + 4 * (16 j + m)
    const int j = m32 >> 4, m = m32 & 15;
    const int ks = c >> 6, kk = c & 63;
    const int lane = m + 16 * (kk >> 4), t = kk & 15;
    tiles[((((static_cast<size_t>(rg) * 4 + rho) * 2 + j) * kss + ks) * 64 + lane) * 16 + t] = w;
  };
  for (const pl::RowGroup& g : L.groups) {
    for (uint32_t j = 0; j < g.count; ++j) {
      put(g.row0, L.ic_index[g.first + j], L.w0[g.first + j]);
      if (g.nrows == 2) put(g.row0 + 1, L.ic_index[g.first + j], L.w1[g.first + j]);
    }
  }
  const hipError_t e = h->wtiles.Upload(tiles.data(), tiles.size());
  if (e != hipSuccess) return FailHip(e, "uploading the weight tiles");
  return PL_OK;
}

// The tiles of the image kernel with one row tile per wavefront: tile w (0 .. 7) of a row group holds rows
// w + 8 m, m = 0 .. 15; [row group][w][k-step][64 lanes][16 bytes], lane l = row m = l % 16, channels
// 64 ks + 16 (l / 16) .. + 15 (image_rows_kernels.hip).
int BuildImageRowsMfma(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int kss = L.ic / 64;
  std::vector<int8_t> tiles(static_cast<size_t>(L.oc) * L.ic, 0);
  auto put = [&](int row, uint32_t c, uint32_t wbits) {
    const int8_t w = static_cast<int8_t>(wbits & 0xffu);
    if (w == 0) return;
    const int rg = row / 128, rl = row % 128;
    const int tile = rl & 7, m = rl >> 3;
    const int ks = c >> 6, kk = c & 63;
    const int lane = m + 16 * (kk >> 4), t = kk & 15;
    tiles[(((static_cast<size_t>(rg) * 8 + tile) * kss + ks) * 64 + lane) * 16 + t] = w;
  };
  for (const pl::RowGroup& g : L.groups) {
    for (uint32_t j = 0; j < g.count; ++j) {
      put(g.row0, L.ic_index[g.first + j], L.w0[g.first + j]);
      if (g.nrows == 2) put(g.row0 + 1, L.ic_index[g.first + j], L.w1[g.first + j]);
    }
  }
  const hipError_t e = h->wtiles_rows.Upload(tiles.data(), tiles.size());
  if (e != hipSuccess) return FailHip(e, "uploading the weight tiles");
  return PL_OK;
}

// The same tiles for the regrouping image kernel where it regroups by transposing LDS reads: byte b of
// lane group g of k-step ks is channel 64 ks + 4 (8 (g % 2) + b % 8) + 2 (b / 8) + g / 2 (image_mfma_kernels.hip).
int BuildImageMfmaTrRegroup(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int kss = L.ic / 64;
  std::vector<int8_t> tiles(static_cast<size_t>(L.oc) * L.ic, 0);
  auto put = [&](int row, uint32_t c, uint32_t wbits) {
    const int8_t w = static_cast<int8_t>(wbits & 0xffu);
    if (w == 0) return;
    const int rg = row / 128, rl = row % 128;
    const int rho = rl & 3, m32 = rl >> 2;  // row = rg * 128 + rho + 4 * (16 j + m)
    const int j = m32 >> 4, m = m32 & 15;
    const int ks = static_cast<int>(c >> 6), cc = static_cast<int>(c & 63u);
    const int par = cc & 1, r = (cc >> 1) & 1, t = cc >> 2;
    const int g = 2 * par + (t >> 3), b = 8 * r + (t & 7);
    const int lane = m + 16 * g;
    tiles[((((static_cast<size_t>(rg) * 4 + rho) * 2 + j) * kss + ks) * 64 + lane) * 16 + b] = w;
  };
  for (const pl::RowGroup& g : L.groups) {
    for (uint32_t j = 0; j < g.count; ++j) {
      put(g.row0, L.ic_index[g.first + j], L.w0[g.first + j]);
      if (g.nrows == 2) put(g.row0 + 1, L.ic_index[g.first + j], L.w1[g.first + j]);
    }
  }
  const hipError_t e = h->wtiles_rg.Upload(tiles.data(), tiles.size());
  if (e != hipSuccess) return FailHip(e, "uploading the weight tiles");
  return PL_OK;
}

// The same tiles for the image kernel with transposing LDS reads.  That kernel
// takes the channels of a k-step in the order its reads deliver them: a step
// holds the 64 channels of one parity out of 128, and byte b of lane group g
// is channel 64 (b / 8) + 4 (8 (g % 2) + b % 8) + 2 (g / 2) + parity of them
// (image_tr_kernels.hip).  Any order is right as long as weights and
// activations agree: the dot product is an exact integer sum.
int BuildImageTrMfma(const pl::DecodedLayout& L, pl_sparse_conv_handle* h) {
  const int steps = L.ic / 64;
  std::vector<int8_t> tiles(static_cast<size_t>(L.oc) * L.ic, 0);
  auto put = [&](int row, uint32_t c, uint32_t wbits) {
    const int8_t w = static_cast<int8_t>(wbits & 0xffu);
    if (w == 0) return;
    const int rg = row / 128, rl = row % 128;
    const int rho = rl & 3, m32 = rl >> 2;  // row = rg * 128 + rho + 4 * (16 j + m)
    const int j = m32 >> 4, m = m32 & 15;
    const int cc = static_cast<int>(c & 127u);
    const int step = 2 * static_cast<int>(c >> 7) + (cc & 1);
    const int u = cc >> 1;            // 32 r + 2 t + (g / 2)
    const int r = u >> 5, t = (u & 31) >> 1, ghi = u & 1;
    const int g = 2 * ghi + (t >> 3), b = 8 * r + (t & 7);
    const int lane = m + 16 * g;
    tiles[((((static_cast<size_t>(rg) * 4 + rho) * 2 + j) * steps + step) * 64 + lane) * 16 + b] = w;
  };
  for (const pl::RowGroup& g : L.groups) {
    for (uint32_t j = 0; j < g.count; ++j) {
      put(g.row0, L.ic_index[g.first + j], L.w0[g.first + j]);
      if (g.nrows == 2) put(g.row0 + 1, L.ic_index[g.first + j], L.w1[g.first + j]);
    }
  }
  const hipError_t e = h->wtiles_tr.Upload(tiles.data(), tiles.size());
  if (e != hipSuccess) return FailHip(e, "uploading the weight tiles");
  return PL_OK;
}

int UploadEpilogue(pl_sparse_conv_handle* h, const float* scale, const float* bias) {
  const size_t n = static_cast<size_t>(h->padded_rows);
  if (scale) {
    std::vector<float> s(n, 0.0f);
    std::copy(scale, scale + h->oc, s.begin());
    hipError_t e = h->scale.Upload(s.data(), n * sizeof(float));
    if (e != hipSuccess) return FailHip(e, "uploading scales");
  }
  if (bias) {
    std::vector<float> b(n, 0.0f);
    std::copy(bias, bias + h->oc, b.begin());
    hipError_t e = h->bias.Upload(b.data(), n * sizeof(float));
    if (e != hipSuccess) return FailHip(e, "uploading biases");
    h->has_bias = true;
  }
  return PL_OK;
}

// Tile shape of the row walk for a given problem.
pl::WalkConfig ChooseWalk(const pl_sparse_conv_handle* h, uint32_t P) {
  pl::WalkConfig c{};
  c.int8 = h->int8;
  c.out_kind = OutKind(h->kind);
  c.nrows = h->semi ? 2 : 1;
  const size_t row_bytes = static_cast<size_t>(h->kd + (h->int8 ? 0 : 1)) * 4;  // fp32 tiles carry a zero row
  // Every workgroup reads its rows' index lists through the scalar cache,
  // whose fill rate is what bounds the walk: wide tiles amortise a list over
  // more positions.  256 positions when two tiles still fit a CU, else 128
  // when one does, else what the channel count leaves room for.
  int tp = 256;
  if (row_bytes * tp > 64 * 1024) tp = 128;
  while (tp > 16 && row_bytes * tp > static_cast<size_t>(pl::kMaxLdsBytes)) tp >>= 1;
  while (tp > 64 && P <= static_cast<uint32_t>(tp) * 8) tp >>= 1;  // small problems: more tiles
  if (h->walk_tile >= 16 && h->walk_tile <= 256 && (h->walk_tile & (h->walk_tile - 1)) == 0 && row_bytes * h->walk_tile <= static_cast<size_t>(pl::kMaxLdsBytes)) tp = h->walk_tile;
  c.tile_pos = tp;
  const size_t lds = row_bytes * tp;
  c.threads = lds > 80 * 1024 ? 1024 : (lds >= 32 * 1024 ? 512 : 256);
  if (c.threads < tp) c.threads = tp;
  const int nwaves = c.threads / 64;
  const uint32_t tiles = (P + tp - 1) / tp;
  int slices = static_cast<int>((1024 + tiles - 1) / tiles);
  slices = std::min(slices, std::max(1, h->n_groups / nwaves));
  slices = std::max(1, std::min(slices, 65535));
  // tuning overrides read at prepare (power-of-two thread counts only)
  if (h->walk_threads >= tp && h->walk_threads <= 1024 && (h->walk_threads & (h->walk_threads - 1)) == 0) c.threads = h->walk_threads;
  if (h->walk_slices > 0) slices = std::max(1, std::min(h->walk_slices, std::max(1, h->n_groups)));
  c.slices = slices;
  return c;
}

// The algorithm one call uses.  Handles prepared for one algorithm use it.  An int8 handle prepared with
// PL_ALGO_AUTO holds the forms of every algorithm its shape allows and picks per call, by what was measured on
// the pointwise shapes of MobileNetV1 at 1 to 64 images per launch:
//  * the image kernels wherever their shape conditions hold: they tie with or beat the block kernel at every
//    batch (by 2x on 7 x 7 maps, where the block kernel has too few tiles for the chip), and stay within 10 % of
//    the row walk on a single 14 x 14 image of 512 channels, the one case where the walk is ahead;
//  * the image kernel with one row tile per wavefront on slabs of larger maps while the slabs are few (below);
//  * else the row walk for at most 256 positions in all (it spreads the output rows over the chip where the
//    block kernel would have one or two tiles);
//  * else the block kernel.
// tuning.image_min_items raises the number of (image, 128-row group) work items the image kernels ask for.
int AlgoForCall(const pl_sparse_conv_handle* h, int batch, int im_size, bool aligned16) {
  if (!h->auto_int8) return h->algo;
  // work items: (image, row group), for 7 x 7 maps (pair of images, row group)
  const int64_t image_items = static_cast<int64_t>(im_size == 49 ? (batch + 1) / 2 : batch) * (h->oc / 128);
  if (h->wtiles.ptr && aligned16 && pl::ImageMfmaFits(h->oc, h->ic, im_size) && image_items >= h->image_min_items) return PL_ALGO_IMAGE_MFMA;
  // Larger maps in slabs of 196 positions: ahead of the block kernel while the slabs are few (128 -> 256 @28x28: 4.0
  // against 4.6 us at 4 images, 4.5 against 5.1 at 16, equal at 64; 256 -> 256 @28x28: 5.3 against 6.0 at 16, 12.7
  // against 10.1 at 64; 128 -> 128 @56x56: 4.3 against 4.7 at 4, 5.9 against 5.5 at 16): every work item pays the
  // kernel's whole load-multiply-store chain, and a CU holds one or two at a time.
  if (h->wtiles_rows.ptr && aligned16 && (h->image_kernel == 0 || h->image_kernel == 3) && pl::ImageRowsSlabFits(h->oc, h->ic, im_size)) {
    const int64_t slab_items = static_cast<int64_t>(batch) * (im_size / 196) * (h->oc / 128);
    if (slab_items >= h->image_min_items && slab_items * 2 <= h->wg_slots_default / 2) return PL_ALGO_IMAGE_MFMA;
  }
  if (h->auto_walk && static_cast<int64_t>(batch) * im_size <= 256) return PL_ALGO_ROW_WALK;
  return h->algo;
}

}  // namespace

extern "C" {

int pl_sparse_conv_abi_version(void) { return PL_SPARSE_CONV_ABI_VERSION; }

const char* pl_last_error(void) { return g_last_error.c_str(); }

int pl_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) {
    (void)hipGetLastError();
    return 0;
  }
  int usable = 0;
  for (int d = 0; d < n; ++d) {
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, d) == hipSuccess && std::strstr(prop.gcnArchName, "gfx950")) ++usable;
  }
  return usable;
}

int pl_sparse_conv_prepare(const pl_sparse_conv_desc* desc, pl_sparse_conv_handle** out_handle) {
  if (!desc || !out_handle) return Fail(PL_ERR_BAD_ARG, "null argument");
  *out_handle = nullptr;
  if (desc->struct_size != sizeof(pl_sparse_conv_desc) && desc->struct_size != offsetof(pl_sparse_conv_desc, tuning))
    return Fail(PL_ERR_BAD_ARG, "pl_sparse_conv_desc size mismatch (%u vs %zu)", desc->struct_size, sizeof(pl_sparse_conv_desc));
  pl_sparse_conv_tuning tune{};
  if (desc->struct_size == sizeof(pl_sparse_conv_desc)) tune = desc->tuning;
  for (int32_t sw : {tune.mfma_stream, tune.mfma_sub_tiles, tune.walk_tiled, tune.walk_chunked, tune.image_tr_regroup, tune.walk_pairs})
    if (sw < PL_TUNE_RULE || sw > PL_TUNE_ALWAYS) return Fail(PL_ERR_BAD_ARG, "a tuning switch is not PL_TUNE_RULE, PL_TUNE_NEVER or PL_TUNE_ALWAYS");
  if (tune.image_kernel < 0 || tune.image_kernel > 3) return Fail(PL_ERR_BAD_ARG, "tuning.image_kernel must be 0, 1, 2 or 3");
  if (desc->kind < PL_KIND_FP32 || desc->kind > PL_KIND_FP16) return Fail(PL_ERR_BAD_ARG, "unknown kind %d", desc->kind);
  if (desc->algo < PL_ALGO_AUTO || desc->algo > PL_ALGO_IMAGE_MFMA) return Fail(PL_ERR_BAD_ARG, "unknown algo %d", desc->algo);
  if (desc->oc <= 0 || desc->ic <= 0 || desc->im_size <= 0) return Fail(PL_ERR_BAD_ARG, "oc, ic and im_size must be positive");
  if (!desc->oc_nonzeros || (desc->n_weights > 0 && (!desc->nonzero_weights || !desc->diffs))) return Fail(PL_ERR_BAD_ARG, "null weight tensors");
  const bool half = desc->kind == PL_KIND_FP16;
  const bool int8 = desc->kind != PL_KIND_FP32 && !half;
  if (int8 && desc->kind != PL_KIND_INT8_ACC32 && !desc->scale) return Fail(PL_ERR_BAD_ARG, "int8 kinds need per-channel scales");
  if ((desc->algo == PL_ALGO_BLOCK_MFMA || desc->algo == PL_ALGO_IMAGE_MFMA) && !int8) return Fail(PL_ERR_UNSUPPORTED, "the MFMA algorithms exist for int8 only");
  if (desc->algo == PL_ALGO_IMAGE_MFMA && !pl::ImageMfmaFits(desc->oc, desc->ic, 16) && !pl::ImageMfmaFits(desc->oc, desc->ic, 49))
    return Fail(PL_ERR_UNSUPPORTED, "the image MFMA algorithm needs oc %% 128 == 0 and ic = 128, 256, 512 or (7 x 7 maps) 1024 (oc = %d, ic = %d)", desc->oc, desc->ic);

  int ndev = 0;
  if (hipGetDeviceCount(&ndev) != hipSuccess || ndev == 0) {
    (void)hipGetLastError();
    return Fail(PL_ERR_NO_DEVICE, "no HIP device: this library has no CPU path");
  }
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return FailHip(e, "hipGetDevice");
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return FailHip(e, "hipGetDeviceProperties");
  if (!std::strstr(prop.gcnArchName, "gfx950")) return Fail(PL_ERR_NO_DEVICE, "device %d is %s; the kernels are built for gfx950 only", dev, prop.gcnArchName);

  pl::DecodedLayout L;
  std::string why;
  if (!pl::DecodeLayout(int8 ? pl::WeightType::kInt8 : pl::WeightType::kFloat, desc->flag_semi != 0, desc->nonzero_weights, desc->n_weights, desc->oc_nonzeros, desc->diffs, desc->n_diffs, desc->first_ic, desc->oc, desc->ic,
                        desc->im_size, &L, &why)) {
    return Fail(PL_ERR_BAD_LAYOUT, "%s", why.c_str());
  }

  pl_sparse_conv_handle* h = new (std::nothrow) pl_sparse_conv_handle();
  if (!h) return Fail(PL_ERR_BAD_ARG, "out of host memory");
  h->device = dev;
  h->wg_slots = 2 * std::max(1, prop.multiProcessorCount);
  h->wg_slots_default = h->wg_slots;
  // tuning overrides (0 = the rule); the switches are kept as 0 never, 1 by rule, 2 whenever possible
  auto sw = [](int32_t t) { return t == PL_TUNE_NEVER ? 0 : (t == PL_TUNE_ALWAYS ? 2 : 1); };
  h->mfma_stream = sw(tune.mfma_stream);
  h->mfma_sub_tiles = sw(tune.mfma_sub_tiles);
  h->walk_tiled = sw(tune.walk_tiled);
  h->walk_pairs = sw(tune.walk_pairs) != 0;  // the rule: pairs
  h->walk_chunked = sw(tune.walk_chunked);
  h->mfma_i8_wide = tune.mfma_narrow_i8_stores == 0;
  if (tune.walk_split > 0) h->walk_split = std::min(kTileWalkSplits, tune.walk_split - 1);
  if (tune.mfma_tile_quads > 0) h->mfma_tile_quads = std::max(8, std::min(32, tune.mfma_tile_quads));
  if (tune.wg_slots > 0) h->wg_slots = tune.wg_slots;
  if (tune.image_min_items > 0) h->image_min_items = tune.image_min_items;
  h->image_kernel = tune.image_kernel;
  h->image_tr_regroup = tune.image_tr_regroup != PL_TUNE_NEVER;
  h->walk_tile = tune.walk_tile;
  h->walk_threads = tune.walk_threads;
  h->walk_slices = tune.walk_slices;
  h->cw_groups = tune.chunk_walk_groups == 4 ? 4 : 8;
  h->kind = desc->kind;
  h->oc = desc->oc;
  h->ic = desc->ic;
  h->int8 = int8;
  h->half = half;
  h->semi = desc->flag_semi != 0;
  h->act = ToDevAct(desc->act);
  h->act_h = ToDevActH(desc->act);
  h->nnz = L.nnz;
  h->stored = L.stored_weights;
  h->entries = static_cast<int64_t>(L.ic_index.size());
  h->padded_rows = CeilDiv(desc->oc, 32) * 32;

  int algo = desc->algo;
  h->auto_int8 = int8 && algo == PL_ALGO_AUTO;
  if (algo == PL_ALGO_AUTO) algo = int8 ? PL_ALGO_BLOCK_MFMA : PL_ALGO_ROW_WALK;
  if (half) {
    // half precision: its own walk; a tile of 16 positions must fit LDS
    if (static_cast<size_t>(desc->ic + 1) * 16 * 2 > static_cast<size_t>(pl::kMaxLdsBytes)) {
      delete h;
      return Fail(PL_ERR_UNSUPPORTED, "ic = %d does not fit an LDS tile", desc->ic);
    }
    h->algo = PL_ALGO_ROW_WALK;
    int hrc = BuildHalfWalk(L, h);
    if (hrc == PL_OK) hrc = BuildChunkWalk(L, h, true);
    // eight positions per lane in the form with the largest tile that holds all channels; the narrow form beside it
    for (int form = 0; hrc == PL_OK && form < pl::kHalfTileWalkNarrowForm; ++form) {
      if (pl::TileWalkLdsBytes(desc->ic, pl::HalfTileWalkTileOf(form) * 2) > static_cast<size_t>(pl::kMaxLdsBytes)) continue;
      h->tw.form = form;
      hrc = BuildTileWalk(L, desc->bias, h, &h->tw, true, pl::HalfTileWalkTileOf(form) * 2, pl::HalfTileWalkGroupsOf(form));
      break;
    }
    h->tw_narrow.form = pl::kHalfTileWalkNarrowForm;
    if (hrc == PL_OK) hrc = BuildTileWalk(L, desc->bias, h, &h->tw_narrow, true, pl::kHalfTileWalkNarrowTile * 2, 2);
    if (hrc == PL_OK) hrc = UploadHalfBias(h, desc->bias);
    if (hrc != PL_OK) {
      delete h;
      return hrc;
    }
    *out_handle = h;
    return PL_OK;
  }
  if (algo == PL_ALGO_ROW_WALK) {
    // fp32 tiles carry one all-zero row behind the channels
    const size_t row_bytes = static_cast<size_t>(int8 ? CeilDiv(desc->ic, 4) : desc->ic + 1) * 4;
    if (row_bytes * 16 > static_cast<size_t>(pl::kMaxLdsBytes)) {
      // the whole-K tile of the plain walk does not fit LDS; the fp32 walk over
      // channel chunks needs no such tile and serves the shapes it supports
      if (int8) {
        delete h;
        return Fail(PL_ERR_UNSUPPORTED, "ic = %d does not fit an LDS tile", desc->ic);
      }
      h->walk_plain_fits = false;
    }
  }
  h->algo = algo;

  const bool mfma_forms = algo == PL_ALGO_BLOCK_MFMA || algo == PL_ALGO_IMAGE_MFMA;
  int rc = PL_OK;
  if (algo == PL_ALGO_ROW_WALK) rc = BuildRowWalk(L, h);
  if (h->auto_int8 && static_cast<size_t>(CeilDiv(desc->ic, 4)) * 4 * 16 <= static_cast<size_t>(pl::kMaxLdsBytes)) {
    rc = BuildRowWalk(L, h);  // for calls of a few hundred positions
    h->auto_walk = rc == PL_OK;
  }
  if (rc == PL_OK && algo == PL_ALGO_BLOCK_MFMA) rc = BuildBlockMfma(L, h);
  if (rc == PL_OK && (algo == PL_ALGO_IMAGE_MFMA || (h->auto_int8 && (pl::ImageMfmaFits(desc->oc, desc->ic, 16) || pl::ImageMfmaFits(desc->oc, desc->ic, 49))))) rc = BuildImageMfma(L, h);
  if (rc == PL_OK && h->wtiles.ptr && pl::ImageTrMfmaFits(desc->oc, desc->ic, 20)) rc = BuildImageTrMfma(L, h);
  if (rc == PL_OK && h->wtiles.ptr && pl::ImageMfmaRegroupsByTransposingReads(desc->ic, 196)) rc = BuildImageMfmaTrRegroup(L, h);
  if (rc == PL_OK && h->wtiles.ptr && pl::ImageRowsMfmaFits(desc->oc, desc->ic, 16)) rc = BuildImageRowsMfma(L, h);
  if (rc == PL_OK && algo == PL_ALGO_ROW_WALK && !int8) rc = BuildChunkWalk(L, h);
  if (rc == PL_OK && algo == PL_ALGO_ROW_WALK && !int8 && !half) {
    // the form with the largest tile that holds all channels in LDS: 128 positions (pairs of row groups, or single
    // ones on request), else 64 / 32 / 16 positions with 4 / 8 / 16 row groups per step
    for (int form = h->walk_pairs ? 1 : 0; form < (h->walk_pairs ? pl::kTileWalkForms : 1); ++form) {
      if (pl::TileWalkLdsBytes(desc->ic, pl::TileWalkTileOf(form) * 4) > static_cast<size_t>(pl::kMaxLdsBytes)) continue;
      h->tw.form = form;
      rc = BuildTileWalk(L, desc->bias, h, &h->tw, false, pl::TileWalkTileOf(form) * 4, pl::TileWalkGroupsOf(form));
      break;
    }
  }
  if (rc == PL_OK) {
    // the MFMA epilogues always read a bias; give them zeros when the op has none
    std::vector<float> zeros;
    const float* bias = desc->bias;
    if (!bias && mfma_forms) {
      zeros.assign(h->oc, 0.0f);
      bias = zeros.data();
    }
    std::vector<float> ones;
    const float* scale = desc->scale;
    if (!scale && int8) {
      ones.assign(h->oc, 1.0f);
      scale = ones.data();
    }
    rc = UploadEpilogue(h, int8 ? scale : nullptr, bias);
    h->has_bias = desc->bias != nullptr || mfma_forms;
  }
  if (rc != PL_OK) {
    delete h;
    return rc;
  }
  *out_handle = h;
  return PL_OK;
}

// From how many positions on a tile walk on tiles of at most 64 positions (more than 271 channels in fp32, more than
// 543 in half precision) is ahead of the plain walk, which loses ground as the channel count grows; measured at 49 -
// 3136 positions on 256 CUs, scaled with the CU count.  Below it a step of 4 - 16 row groups leaves a wavefront too
// few, too long units.
bool SmallTilesPay(const pl_sparse_conv_handle* h, int tile, uint32_t P) {
  const int64_t from = tile >= 64 ? (h->semi ? 1024 : 640) : (h->semi ? 784 : 392);
  return static_cast<int64_t>(P) * 512 >= from * h->wg_slots_default;
}

// How a tile walk of `tiles` tiles is divided over the CUs, and where the stream tables of that division start.
// With fewer tiles than CUs, the CUs without a tile take a share of the row groups of several tiles each
// (one after the other, each staged anew).  The share that evens out the two kinds of workgroup: a main
// workgroup spends S + (1 - f) W, a spare one r (S + f W) for its r tiles, with S the staging time of a tile
// and W the walk of all row groups, so f = (1 - (r - 1) S / W) / (r + 1).  S and W in cycles, fitted to
// measurements (a tile of 256 channels costs a spare workgroup about 5.6 K cycles besides its walk; 355
// cycles per work unit of the fullest stream).  Rounded down: a share above the balance point costs r
// times what one below it costs.
struct TileWalkDivision {
  int split = 0;    // 0 none, 1 main + spare part, 2 equal parts
  int parts = 0;    // equal parts
  int split_slots = 0;
  size_t table = 0;  // first entry of the division's stream tables
};

TileWalkDivision DivideTileWalk(const pl_sparse_conv_handle* h, const TileWalkStreams& tw, int tiles) {
  TileWalkDivision d;
  const int cus = std::max(8, h->wg_slots_default / 2) / 8 * 8;
  int s16 = 0, equal_parts = 0;
  if (tiles < cus && h->walk_split != 0) {
    const int per_xcd = CeilDiv(tiles, 8), spare = cus / 8 - per_xcd;
    if (h->walk_split < 0 && per_xcd * 3 <= cus / 8) {
      // at most a third as many tiles as CUs: n workgroups per tile, equal shares
      const int room = (cus / 8) / per_xcd;
      for (int n : kTileWalkEqualParts)
        if (n <= room) equal_parts = n;
    } else if (spare >= 1) {
      const int r = CeilDiv(per_xcd, spare);
      const double sw = (2000.0 + 14.0 * h->ic) / (355.0 * static_cast<double>(std::max<int64_t>(1, tw.stream_work)));
      const double f = (1.0 - (r - 1) * sw) / (r + 1);
      s16 = h->walk_split > 0 ? h->walk_split : static_cast<int>(f * 16.0 + 0.3);
      s16 = std::max(0, std::min(kTileWalkSplits, s16));
    }
  }
  // stream tables: set 0 has one part, sets 1 .. 8 two, then the equal divisions
  d.table = s16 == 0 ? 0 : static_cast<size_t>(pl::kTileWalkWaves) * (2 * s16 - 1);
  if (equal_parts != 0) {
    d.table = static_cast<size_t>(pl::kTileWalkWaves) * (1 + 2 * kTileWalkSplits);
    for (int n : kTileWalkEqualParts) {
      if (n == equal_parts) break;
      d.table += static_cast<size_t>(pl::kTileWalkWaves) * n;
    }
  }
  d.split = equal_parts != 0 ? 2 : (s16 != 0 ? 1 : 0);
  d.parts = equal_parts;
  d.split_slots = cus / 8;
  return d;
}

int pl_sparse_conv_run(pl_sparse_conv_handle* h, const void* x_dev, void* out_dev, int32_t batch, int32_t im_size, void* stream) {
  if (!h) return Fail(PL_ERR_BAD_ARG, "null handle");
  if (batch < 0 || im_size <= 0) return Fail(PL_ERR_BAD_ARG, "batch must be >= 0 and im_size > 0");
  if (batch == 0) return PL_OK;
  if (!x_dev || !out_dev) return Fail(PL_ERR_BAD_ARG, "null device pointer");
  int cur_dev = -1;
  if (hipGetDevice(&cur_dev) != hipSuccess || cur_dev != h->device) return Fail(PL_ERR_BAD_ARG, "the handle belongs to device %d, the current device is %d", h->device, cur_dev);
  const int64_t P64 = static_cast<int64_t>(batch) * im_size;
  if (P64 >= (1ll << 31) - 512) return Fail(PL_ERR_UNSUPPORTED, "batch * im_size = %lld exceeds 2^31", static_cast<long long>(P64));
  const uint32_t P = static_cast<uint32_t>(P64);
  const int vec = (im_size % 4 == 0) && (reinterpret_cast<uintptr_t>(x_dev) % 16 == 0) && (reinterpret_cast<uintptr_t>(out_dev) % 16 == 0);
  const bool aligned16 = reinterpret_cast<uintptr_t>(x_dev) % 16 == 0 && reinterpret_cast<uintptr_t>(out_dev) % 16 == 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipError_t e;
  const int call_algo = AlgoForCall(h, batch, im_size, aligned16);
  // Half precision: the walk with the tile and the lists in LDS, from 7 tiles on (13 with row pairs, whose plain
  // walk is twice as efficient per list entry) on 256 CUs: measured against the other half-precision walks at
  // 1 - 784 tiles, it is 1.3 - 2.5 times as fast from there on and slower below.  Tiles of 256 positions where
  // the channels fit and the map size is a multiple of 8, else tiles of 128.
  const bool aligned8 = reinterpret_cast<uintptr_t>(x_dev) % 8 == 0 && reinterpret_cast<uintptr_t>(out_dev) % 8 == 0;
  const TileWalkStreams* half_tw = nullptr;
  int half_tile = 0;
  bool half_ragged = false;
  if (h->half && h->walk_tiled > 0) {
    if (h->tw.built != 0 && im_size % 8 == 0 && aligned16) {
      half_tw = &h->tw;
    } else if (h->tw_narrow.built != 0 && im_size % 4 == 0 && aligned8) {
      half_tw = &h->tw_narrow;
    } else if (reinterpret_cast<uintptr_t>(x_dev) % 2 == 0 && reinterpret_cast<uintptr_t>(out_dev) % 2 == 0 && (h->tw.built != 0 || h->tw_narrow.built != 0)) {
      // any other map size or alignment: value by value in and out of the tile
      half_tw = h->tw.built != 0 ? &h->tw : &h->tw_narrow;
      half_ragged = true;
    }
    if (half_tw) half_tile = pl::HalfTileWalkTileOf(half_tw->form);
    if (half_tw && h->walk_tiled != 2) {
      const bool pays = half_tile <= 64 ? SmallTilesPay(h, 32, P) : (h->semi ? 42 : 84) * static_cast<int64_t>(CeilDiv(static_cast<int>(P), half_tile)) >= h->wg_slots_default;
      if (!pays) half_tw = nullptr;
    }
  }
  if (half_tw) {
    const TileWalkDivision d = DivideTileWalk(h, *half_tw, CeilDiv(static_cast<int>(P), half_tile));
    pl::HalfTileWalkParams p{};
    p.x = static_cast<const uint16_t*>(x_dev);
    p.out = static_cast<uint16_t*>(out_dev);
    p.stream = half_tw->stream.ptr;
    p.stream_first = static_cast<const uint32_t*>(half_tw->first.ptr) + d.table;
    p.stream_groups = static_cast<const uint32_t*>(half_tw->desc.ptr) + d.table;
    p.split = static_cast<int16_t>(d.split);
    p.parts = static_cast<int8_t>(d.parts);
    p.form = static_cast<int8_t>(half_tw->form | (half_ragged ? pl::kTileWalkRagged : 0));
    p.split_slots = d.split_slots;
    p.n_groups = h->n_groups;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.act = h->act_h;
    e = pl::LaunchHalfTileWalk(h->semi ? 2 : 1, p, s);
  } else if (h->half && (im_size % 4 == 0) && (reinterpret_cast<uintptr_t>(x_dev) % 8 == 0) && (reinterpret_cast<uintptr_t>(out_dev) % 8 == 0) && h->walk_chunked > 0 && h->cw_chunks > 0 &&
      (h->walk_chunked == 2 || (h->ic > 128 && static_cast<int64_t>(CeilDiv(static_cast<int>(P), pl::kChunkWalkTile)) * h->cw_slices >= 256))) {
    // many channels and enough work for every CU: walk over channel chunks
    pl::HalfChunkWalkParams p{};
    p.x = static_cast<const uint16_t*>(x_dev);
    p.out = static_cast<uint16_t*>(out_dev);
    p.groups = static_cast<const pl::DevGroup*>(h->groups.ptr);
    p.desc = static_cast<const uint32_t*>(h->cw_desc.ptr);
    p.idx = static_cast<const uint32_t*>(h->cw_idx.ptr);
    p.wts = static_cast<const uint32_t*>(h->cw_wts.ptr);
    p.bias = h->has_bias ? static_cast<const uint16_t*>(h->hw_bias.ptr) : nullptr;
    p.n_groups = h->n_groups;
    p.n_chunks = h->cw_chunks;
    p.slices = h->cw_slices;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.act = h->act_h;
    e = pl::LaunchHalfChunkWalk(h->semi ? 2 : 1, p, s);
  } else if (h->half) {
    pl::HalfWalkParams p{};
    p.x = static_cast<const uint16_t*>(x_dev);
    p.out = static_cast<uint16_t*>(out_dev);
    p.groups = static_cast<const pl::DevGroup*>(h->groups.ptr);
    p.kidx = static_cast<const uint32_t*>(h->hw_kidx.ptr);
    p.wts = static_cast<const uint32_t*>(h->hw_wts.ptr);
    p.bias = h->has_bias ? static_cast<const uint16_t*>(h->hw_bias.ptr) : nullptr;
    p.n_groups = h->n_groups;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.pair = (im_size % 2 == 0) && (reinterpret_cast<uintptr_t>(x_dev) % 4 == 0) && (reinterpret_cast<uintptr_t>(out_dev) % 4 == 0);
    p.act = h->act_h;
    // widest tile of which two fit a CU, else the widest that fits at all
    const size_t row_bytes = static_cast<size_t>(h->ic + 1) * 2;
    int tp = 128;
    while (tp > 16 && row_bytes * tp > 64 * 1024) tp >>= 1;
    if (row_bytes * tp > 64 * 1024) {
      tp = 128;
      while (tp > 16 && row_bytes * tp > static_cast<size_t>(pl::kMaxLdsBytes)) tp >>= 1;
    }
    const int threads = row_bytes * tp > 32 * 1024 ? 512 : 256;
    const uint32_t tiles = (P + tp - 1) / tp;
    int slices = static_cast<int>((1024 + tiles - 1) / tiles);
    slices = std::max(1, std::min(slices, std::max(1, h->n_groups / (threads / 64))));
    p.groups_per_slice = CeilDiv(h->n_groups, slices);
    p.slices = CeilDiv(h->n_groups, p.groups_per_slice);
    e = pl::LaunchHalfWalk(h->semi ? 2 : 1, tp, threads, p, s);
  } else if (call_algo == PL_ALGO_IMAGE_MFMA) {
    // larger maps of a multiple of 196 positions are taken slab by slab by the kernel with one row tile per wavefront
    const bool slabs = h->wtiles_rows.ptr != nullptr && (h->image_kernel == 0 || h->image_kernel == 3) && pl::ImageRowsSlabFits(h->oc, h->ic, im_size);
    if (!slabs && !pl::ImageMfmaFits(h->oc, h->ic, im_size))
      return Fail(PL_ERR_UNSUPPORTED, "the image MFMA algorithm needs H*W = 49, a multiple of 4 in [16, 256] or a multiple of 196 (its slabs) that fits LDS with %d channels (H*W = %d)", h->ic, im_size);
    if (reinterpret_cast<uintptr_t>(x_dev) % 16 != 0 || reinterpret_cast<uintptr_t>(out_dev) % 16 != 0) return Fail(PL_ERR_UNSUPPORTED, "the image MFMA algorithm needs 16-byte aligned tensors");
    pl::ImageMfmaParams p{};
    p.x = static_cast<const int8_t*>(x_dev);
    p.out = out_dev;
    p.scale = static_cast<const float*>(h->scale.ptr);
    p.bias = static_cast<const float*>(h->bias.ptr);
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.batch = batch;
    p.act = h->act;
    // The kernel with transposing LDS reads runs on request only: on 64 x 512 -> 512 @14x14 it is about 4 %
    // slower than the kernel that regroups the image (9.9 against 9.7 us).
    const bool tr_fits = h->wtiles_tr.ptr != nullptr && pl::ImageTrMfmaFits(h->oc, h->ic, im_size);
    // One row tile per wavefront and the image through registers: the rule wherever it applies (every shape of
    // the image algorithm but the 7 x 7 maps).
    const bool rows_fits = h->wtiles_rows.ptr != nullptr && (slabs || pl::ImageRowsMfmaFits(h->oc, h->ic, im_size));
    if (h->image_kernel == 3 && !rows_fits) return Fail(PL_ERR_UNSUPPORTED, "the image kernel with one row tile per wavefront takes no 7 x 7 maps (H*W = %d, ic = %d)", im_size, h->ic);
    if (h->image_kernel == 2 && !tr_fits) return Fail(PL_ERR_UNSUPPORTED, "the image kernel with transposing LDS reads needs H*W = 4 (mod 8) from 20 on, ic = 128, 256 or 512 and an image that leaves 41 KB of LDS free (H*W = %d, ic = %d)", im_size, h->ic);
    if (tr_fits && h->image_kernel == 2) {
      p.wtiles = h->wtiles_tr.ptr;
      e = pl::LaunchImageTrMfma(OutKind(h->kind), p, s);
    } else if (rows_fits && (h->image_kernel == 0 || h->image_kernel == 3)) {
      p.wtiles = h->wtiles_rows.ptr;
      e = pl::LaunchImageRowsMfma(OutKind(h->kind), p, s);
    } else {
      p.tr_regroup = h->image_tr_regroup && h->wtiles_rg.ptr != nullptr && pl::ImageMfmaRegroupsByTransposingReads(h->ic, im_size);
      p.wtiles = p.tr_regroup ? h->wtiles_rg.ptr : h->wtiles.ptr;
      e = pl::LaunchImageMfma(OutKind(h->kind), p, s);
    }
  } else if (call_algo == PL_ALGO_BLOCK_MFMA) {
    pl::MfmaParams p{};
    p.x = static_cast<const int8_t*>(x_dev);
    p.out = out_dev;
    p.wblocks = h->wblocks.ptr;
    p.kmask = static_cast<const uint32_t*>(h->kmask.ptr);
    p.kmask_words = h->kmask_words;
    p.scale = static_cast<const float*>(h->scale.ptr);
    p.bias = static_cast<const float*>(h->bias.ptr);
    p.row_blocks = h->row_blocks;
    p.ksteps = h->ksteps;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.small = (P64 * h->ic < (1ll << 31)) && (P64 * h->oc * 4 < (1ll << 31));
    p.act = h->act;
    pl::MfmaConfig c{};
    c.out_kind = OutKind(h->kind);
    c.ks_max = 2;
    while (c.ks_max < h->ksteps && c.ks_max < 64) c.ks_max <<= 1;  // 64: any count, a chunk at a time
    // Tile width: full 128-position tiles unless that leaves CUs without a
    // workgroup (narrower tiles measured slower on the 392-workgroup metric
    // shape: every workgroup pays for its own copy of the weight blocks).
    const int row_groups = CeilDiv(h->row_blocks, 4);
    const int64_t quads = static_cast<int64_t>(batch) * ((im_size + 3) / 4);
    const int64_t full_tiles = (quads + 31) / 32;
    c.tile_quads = 32;
    if (full_tiles * row_groups < h->wg_slots / 2) {
      const int64_t target_tiles = std::max<int64_t>(1, (h->wg_slots / 2) / row_groups);
      c.tile_quads = static_cast<int>(std::min<int64_t>(32, std::max<int64_t>(8, (quads + target_tiles - 1) / target_tiles)));
    }
    c.i8_wide_stores = h->mfma_i8_wide;
    c.stream = h->mfma_stream;
    c.cus = std::max(1, h->wg_slots_default / 2);
    c.sub_tiles = h->mfma_sub_tiles;
    if (h->mfma_tile_quads > 0) c.tile_quads = h->mfma_tile_quads;
    e = pl::LaunchBlockMfma(c, p, s);
  } else if (!h->int8 && !h->half && h->tw.built != 0 && h->walk_tiled > 0 &&
             (vec || (h->tw.form != 0 && reinterpret_cast<uintptr_t>(x_dev) % 4 == 0 && reinterpret_cast<uintptr_t>(out_dev) % 4 == 0)) &&
             (h->walk_tiled == 2 || (vec ? (h->tw.form >= 2 ? SmallTilesPay(h, pl::TileWalkTileOf(h->tw.form), P) : 32 * static_cast<int64_t>(CeilDiv(static_cast<int>(P), pl::kTileWalkTile)) >= h->wg_slots_default)
                                         // the other walks move such tensors element by element too and lose earlier: measured
                                         // crossover at 400 - 700 positions with row pairs, 50 - 200 without (256 CUs)
                                         : (h->semi ? 4 : 14) * static_cast<int64_t>(P) >= 5 * static_cast<int64_t>(h->wg_slots_default)))) {
    // fp32 with tiles for at least a sixteenth of the CUs (the
    // row groups of a tile are shared between up to ten CUs; measured
    // crossover against the other walks between 13 and 25 tiles on 256 CUs):
    // the walk with the tile and the lists in LDS, in the form the streams were made for (tiles of 128 positions, or
    // smaller ones where only those hold all channels); element by element in and out of the tile where the map
    // size is not a multiple of 4 or the tensors are not 16-byte aligned
    const TileWalkStreams& tw = h->tw;
    const int tile = pl::TileWalkTileOf(tw.form);
    pl::TileWalkParams p{};
    p.x = static_cast<const float*>(x_dev);
    p.out = static_cast<float*>(out_dev);
    p.stream = tw.stream.ptr;
    const TileWalkDivision d = DivideTileWalk(h, tw, CeilDiv(static_cast<int>(P), tile));
    p.stream_first = static_cast<const uint32_t*>(tw.first.ptr) + d.table;
    p.stream_groups = static_cast<const uint32_t*>(tw.desc.ptr) + d.table;
    p.split = static_cast<int16_t>(d.split);
    p.parts = static_cast<int8_t>(d.parts);
    p.pairs = static_cast<int8_t>(tw.form | (vec ? 0 : pl::kTileWalkRagged));
    p.split_slots = d.split_slots;
    p.n_groups = h->n_groups;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.act = h->act;
    e = pl::LaunchTileWalk(h->semi ? 2 : 1, p, s);
  } else if (!h->int8 && !h->walk_plain_fits && !vec) {
    return Fail(PL_ERR_UNSUPPORTED, "fp32 with ic = %d runs as a walk over channel chunks, which needs H*W %% 4 == 0 and 16-byte aligned tensors (H*W = %d)", h->ic, im_size);
  } else if (!h->int8 && vec && h->cw_chunks > 0 &&
             (!h->walk_plain_fits || (h->walk_chunked > 0 && (h->walk_chunked == 2 || (h->ic > 128 && static_cast<int64_t>(CeilDiv(static_cast<int>(P), pl::kChunkWalkTile)) * h->cw_slices >= 256))))) {
    // fp32 with many channels and enough work for every CU: walk over
    // channel chunks (256 positions per list fetch)
    pl::ChunkWalkParams p{};
    p.x = x_dev;
    p.out = out_dev;
    p.groups = static_cast<const pl::DevGroup*>(h->groups.ptr);
    p.desc = static_cast<const uint32_t*>(h->cw_desc.ptr);
    p.idx = static_cast<const uint32_t*>(h->cw_idx.ptr);
    p.wts = static_cast<const uint32_t*>(h->cw_wts.ptr);
    p.bias = h->has_bias ? static_cast<const float*>(h->bias.ptr) : nullptr;
    p.n_groups = h->n_groups;
    p.n_chunks = h->cw_chunks;
    p.slices = h->cw_slices;
    p.groups_per_wave = h->cw_groups;
    p.M = h->oc;
    p.K = h->ic;
    p.hw = im_size;
    p.P = P;
    p.act = h->act;
    e = pl::LaunchChunkWalk(h->semi ? 2 : 1, p, s);
  } else {
    pl::WalkParams p{};
    p.x = x_dev;
    p.out = out_dev;
    p.groups = static_cast<const pl::DevGroup*>(h->groups.ptr);
    p.kidx = static_cast<const uint32_t*>(h->kidx.ptr);
    p.wts = static_cast<const uint32_t*>(h->wts.ptr);
    p.scale = static_cast<const float*>(h->scale.ptr);
    p.bias = h->has_bias ? static_cast<const float*>(h->bias.ptr) : nullptr;
    p.n_groups = h->n_groups;
    p.M = h->oc;
    p.K = h->ic;
    p.kd = h->kd;
    p.hw = im_size;
    p.P = P;
    p.vec = vec;
    p.act = h->act;
    pl::WalkConfig c = ChooseWalk(h, P);
    p.groups_per_slice = CeilDiv(h->n_groups, c.slices);
    c.slices = CeilDiv(h->n_groups, p.groups_per_slice);
    e = pl::LaunchRowWalk(c, p, s);
  }
  if (e != hipSuccess) return FailHip(e, "kernel launch");
  return PL_OK;
}

int pl_sparse_conv_run_sequence(pl_sparse_conv_handle* h, const void* const* x_dev, void* const* out_dev, int32_t n_sets, int32_t batch, int32_t im_size, int32_t steps, void* stream, float* elapsed_ms) {
  if (!h || !x_dev || !out_dev || n_sets <= 0 || steps < 0) return Fail(PL_ERR_BAD_ARG, "bad sequence arguments");
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipEvent_t t0 = nullptr, t1 = nullptr;
  if (elapsed_ms) {
    hipError_t e = hipEventCreate(&t0);
    if (e == hipSuccess) e = hipEventCreate(&t1);
    if (e == hipSuccess) e = hipEventRecord(t0, s);
    if (e != hipSuccess) {
      if (t0) (void)hipEventDestroy(t0);
      if (t1) (void)hipEventDestroy(t1);
      return FailHip(e, "creating timing events");
    }
  }
  int rc = PL_OK;
  for (int i = 0; i < steps && rc == PL_OK; ++i) rc = pl_sparse_conv_run(h, x_dev[i % n_sets], out_dev[i % n_sets], batch, im_size, stream);
  if (elapsed_ms) {
    hipError_t e = hipEventRecord(t1, s);
    if (e == hipSuccess) e = hipEventSynchronize(t1);
    if (e == hipSuccess) e = hipEventElapsedTime(elapsed_ms, t0, t1);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    if (rc == PL_OK && e != hipSuccess) rc = FailHip(e, "timing the sequence");
  }
  return rc;
}

int pl_sparse_conv_get_info(const pl_sparse_conv_handle* h, pl_sparse_conv_info* info) {
  if (!h || !info) return Fail(PL_ERR_BAD_ARG, "null argument");
  std::memset(info, 0, sizeof(*info));
  info->algo = h->algo;
  info->oc = h->oc;
  info->ic = h->ic;
  info->nnz = h->nnz;
  info->stored_weights = h->stored;
  info->index_entries = h->entries;
  info->device_bytes = h->DeviceBytes();
  info->mfma_blocks = h->blocks_present;
  info->mfma_blocks_total = static_cast<int64_t>(h->row_blocks) * h->ksteps;
  return PL_OK;
}

int pl_sparse_conv_algo_for(const pl_sparse_conv_handle* h, int32_t batch, int32_t im_size) {
  if (!h) return Fail(PL_ERR_BAD_ARG, "null handle");
  if (batch < 0 || im_size <= 0) return Fail(PL_ERR_BAD_ARG, "batch must be >= 0 and im_size > 0");
  return AlgoForCall(h, batch, im_size, true);
}

int pl_sparse_conv_set_epilogue(pl_sparse_conv_handle* h, const float* scale, const float* bias, const pl_activation* act) {
  if (!h) return Fail(PL_ERR_BAD_ARG, "null handle");
  if (scale && !h->int8) return Fail(PL_ERR_BAD_ARG, "floating-point kernels take no scales");
  int rc = h->half ? UploadHalfBias(h, bias) : UploadEpilogue(h, scale, bias);
  if (rc != PL_OK) return rc;
  for (TileWalkStreams* tw : {&h->tw, &h->tw_narrow}) {
    if (!bias || !tw->built) continue;
    // the tile walk starts its accumulators from the bias in its header records
    for (const auto& slot : tw->bias_slots) {
      const uint32_t row0 = slot.second & 0xffffffu, nrows = slot.second >> 24;
      uint32_t b0 = 0, b1 = 0;
      std::memcpy(&b0, &bias[row0], 4);
      if (nrows == 2) std::memcpy(&b1, &bias[row0 + 1], 4);
      tw->host_stream[slot.first] = h->half ? DoubledHalf(b0) : b0;
      if (nrows == 2) tw->host_stream[slot.first + 1] = h->half ? DoubledHalf(b1) : b1;
    }
    const hipError_t e = tw->stream.Upload(tw->host_stream.data(), tw->host_stream.size() * sizeof(uint32_t));
    if (e != hipSuccess) return FailHip(e, "uploading the tile-walk list streams");
  }
  if (act) {
    h->act = ToDevAct(*act);
    h->act_h = ToDevActH(*act);
  }
  return PL_OK;
}

void pl_sparse_conv_destroy(pl_sparse_conv_handle* h) { delete h; }

int pl_fp32_to_fp16(const float* in, uint16_t* out, int64_t n) {
  if (n < 0 || (n > 0 && (!in || !out))) return Fail(PL_ERR_BAD_ARG, "bad conversion arguments");
  for (int64_t i = 0; i < n; ++i) out[i] = HalfBits(in[i]);
  return PL_OK;
}

namespace {
int CheckCalibArgs(const void* x, const void* out, int64_t n, float scale) {
  if (n < 0) return Fail(PL_ERR_BAD_ARG, "negative element count");
  if (n > 0 && (!x || !out)) return Fail(PL_ERR_BAD_ARG, "null device pointer");
  if (!(scale > 0.0f) || !std::isfinite(scale)) return Fail(PL_ERR_BAD_ARG, "scale must be positive and finite");
  static const int devices = pl_device_count();  // looked up once per process
  if (n > 0 && devices == 0) return Fail(PL_ERR_NO_DEVICE, "no gfx950 device");
  return PL_OK;
}
}  // namespace

int pl_calib_fp32_to_int8(const float* x_dev, int8_t* out_dev, int64_t n, float scale, void* stream) {
  const int rc = CheckCalibArgs(x_dev, out_dev, n, scale);
  if (rc != PL_OK || n == 0) return rc;
  const hipError_t e = pl::LaunchFp32ToInt8(x_dev, out_dev, n, scale, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? PL_OK : FailHip(e, "fp32 -> int8 launch");
}

int pl_calib_int8_to_fp32(const int8_t* x_dev, float* out_dev, int64_t n, float scale, void* stream) {
  const int rc = CheckCalibArgs(x_dev, out_dev, n, scale);
  if (rc != PL_OK || n == 0) return rc;
  const hipError_t e = pl::LaunchInt8ToFp32(x_dev, out_dev, n, scale, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? PL_OK : FailHip(e, "int8 -> fp32 launch");
}

// ------------------------------------------------------------ host packers
int pl_sparse_count_semi(int32_t dtype, const void* dense, int32_t oc, int32_t ic, int32_t* count_nonzeroes, int32_t* count_channels, int32_t* count_blocks, int32_t* flag_semi) {
  if (!dense || oc <= 0 || ic <= 0 || (dtype != 0 && dtype != 1)) return Fail(PL_ERR_BAD_ARG, "bad argument");
  pl::SemiCounts c = dtype == 0 ? pl::CountSemi(static_cast<const float*>(dense), oc, ic) : pl::CountSemi(static_cast<const int8_t*>(dense), oc, ic);
  if (count_nonzeroes) *count_nonzeroes = c.count_nonzeroes;
  if (count_channels) *count_channels = c.count_channels;
  if (count_blocks) *count_blocks = c.count_blocks;
  if (flag_semi) *flag_semi = c.flag_semi;
  return c.zeros;
}

int pl_sparse_count_zeros(int32_t dtype, const void* dense, int32_t oc, int32_t ic, int32_t* num_build_nonzeroes) {
  if (!dense || oc <= 0 || ic <= 0 || (dtype != 0 && dtype != 1)) return Fail(PL_ERR_BAD_ARG, "bad argument");
  int nb = 0;
  int z = dtype == 0 ? pl::CountZerosPad4(static_cast<const float*>(dense), oc, ic, &nb) : pl::CountZerosPad4(static_cast<const int8_t*>(dense), oc, ic, &nb);
  if (num_build_nonzeroes) *num_build_nonzeroes = nb;
  return z;
}

int pl_sparse_pack(int32_t dtype, int32_t flag_semi, const void* dense, int32_t oc, int32_t ic, int32_t im_size, void* nonzero_weights, int64_t n_weights, uint32_t* oc_nonzeros, int32_t* diffs, int64_t n_diffs) {
  if (!dense || !oc_nonzeros || oc <= 0 || ic <= 0 || im_size <= 0 || (dtype != 0 && dtype != 1)) return Fail(PL_ERR_BAD_ARG, "bad argument");
  // the arrays must have exactly the sizes the counting passes report
  int64_t need_w = 0, need_d = 0;
  if (flag_semi) {
    pl::SemiCounts c = dtype == 0 ? pl::CountSemi(static_cast<const float*>(dense), oc, ic) : pl::CountSemi(static_cast<const int8_t*>(dense), oc, ic);
    if (!c.flag_semi) {
      // caller forces the paired layout on a matrix the rule would not pick:
      // count its blocks directly
      int64_t blocks = 0, tail = 0;
      const int even = oc - (oc & 1);
      for (int r = 0; r < even; r += 2)
        for (int k = 0; k < ic; ++k) {
          bool a, b;
          if (dtype == 0) {
            const float* w = static_cast<const float*>(dense);
            a = w[(size_t)r * ic + k] != 0.f;
            b = w[(size_t)(r + 1) * ic + k] != 0.f;
          } else {
            const int8_t* w = static_cast<const int8_t*>(dense);
            a = w[(size_t)r * ic + k] != 0;
            b = w[(size_t)(r + 1) * ic + k] != 0;
          }
          blocks += (a || b);
        }
      for (int r = even; r < oc; ++r)
        for (int k = 0; k < ic; ++k) tail += dtype == 0 ? (static_cast<const float*>(dense)[(size_t)r * ic + k] != 0.f) : (static_cast<const int8_t*>(dense)[(size_t)r * ic + k] != 0);
      need_w = 2 * blocks + tail;
      need_d = blocks + tail;
    } else {
      need_w = c.count_nonzeroes;
      need_d = c.count_blocks;
    }
  } else if (dtype == 0) {
    int nb = 0;
    pl::CountZerosPad4(static_cast<const float*>(dense), oc, ic, &nb);
    need_w = need_d = nb;
  } else {
    int nb = 0;
    int z = pl::CountZerosPad4(static_cast<const int8_t*>(dense), oc, ic, &nb);
    need_w = need_d = static_cast<int64_t>(oc) * ic - z;
  }
  if (n_weights != need_w || n_diffs != need_d) return Fail(PL_ERR_BAD_ARG, "output arrays must hold %lld weights and %lld diffs", static_cast<long long>(need_w), static_cast<long long>(need_d));
  if (need_w > 0 && (!nonzero_weights || !diffs)) return Fail(PL_ERR_BAD_ARG, "null output array");
  std::memset(oc_nonzeros, 0, sizeof(uint32_t) * oc);  // semi writes only oc/2 + oc%2 entries
  if (dtype == 0) return pl::PackWeights(static_cast<const float*>(dense), oc, ic, im_size, flag_semi != 0, static_cast<float*>(nonzero_weights), oc_nonzeros, diffs);
  return pl::PackWeights(static_cast<const int8_t*>(dense), oc, ic, im_size, flag_semi != 0, static_cast<int8_t*>(nonzero_weights), oc_nonzeros, diffs);
}

// ------------------------------------------------ depthwise 3x3 convolution
struct pl_dwconv_handle {
  int device = 0;
  int kind = 0, channels = 0, stride = 1, pad = 0;
  DevBuf wpack, scale, bias;
  pl::DevAct act{};
  int item_rows = 0;     // 0 = chosen per shape
  int item_cols = 0;     // 0 = chosen per shape
  int share_lanes = -1;  // -1 = chosen per shape, 0 / 1 forced
  int row_items = -1;    // -1 = chosen per shape, 0 / 1 forced
};

int pl_dwconv3x3_prepare(const pl_dwconv_desc* desc, pl_dwconv_handle** out_handle) {
  if (!desc || !out_handle) return Fail(PL_ERR_BAD_ARG, "null argument");
  *out_handle = nullptr;
  if (desc->struct_size != sizeof(pl_dwconv_desc) && desc->struct_size != offsetof(pl_dwconv_desc, item_rows))
    return Fail(PL_ERR_BAD_ARG, "pl_dwconv_desc size mismatch (%u vs %zu)", desc->struct_size, sizeof(pl_dwconv_desc));
  const bool tuned = desc->struct_size == sizeof(pl_dwconv_desc);
  if (tuned && (desc->share_lanes < PL_TUNE_RULE || desc->share_lanes > PL_TUNE_ALWAYS || desc->row_items < PL_TUNE_RULE || desc->row_items > PL_TUNE_ALWAYS))
    return Fail(PL_ERR_BAD_ARG, "a tuning switch is not PL_TUNE_RULE, PL_TUNE_NEVER or PL_TUNE_ALWAYS");
  if (desc->kind != PL_KIND_INT8_FP32 && desc->kind != PL_KIND_INT8_INT8) return Fail(PL_ERR_BAD_ARG, "kind must be int8 -> fp32 or int8 -> int8");
  if (desc->channels <= 0) return Fail(PL_ERR_BAD_ARG, "channels must be positive");
  if (desc->stride != 1 && desc->stride != 2) return Fail(PL_ERR_UNSUPPORTED, "stride %d: only 1 and 2 exist", desc->stride);
  if (desc->pad != 0 && desc->pad != 1) return Fail(PL_ERR_UNSUPPORTED, "padding %d: only 0 and 1 exist", desc->pad);
  if (!desc->weights || !desc->scale) return Fail(PL_ERR_BAD_ARG, "null weights or scales");
  switch (desc->act.type) {
    case PL_ACT_NONE:
    case PL_ACT_RELU:
    case PL_ACT_RELU6:
    case PL_ACT_LEAKY_RELU:
    case PL_ACT_HARD_SWISH:
      break;
    default:
      return Fail(PL_ERR_UNSUPPORTED, "activation %d has no kernel", desc->act.type);
  }
  if (pl_device_count() == 0) return Fail(PL_ERR_NO_DEVICE, "no gfx950 device: this library has no CPU path");
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return FailHip(e, "hipGetDevice");
  hipDeviceProp_t prop;
  e = hipGetDeviceProperties(&prop, dev);
  if (e != hipSuccess) return FailHip(e, "hipGetDeviceProperties");
  if (!std::strstr(prop.gcnArchName, "gfx950")) return Fail(PL_ERR_NO_DEVICE, "device %d is %s; the kernels are built for gfx950 only", dev, prop.gcnArchName);

  std::unique_ptr<pl_dwconv_handle> h(new pl_dwconv_handle);
  h->device = dev;
  h->kind = desc->kind;
  h->channels = desc->channels;
  h->stride = desc->stride;
  h->pad = desc->pad;
  h->act = ToDevAct(desc->act);
  h->act.hs_inv_scale = desc->act.hs_scale;  // this op multiplies by the scale itself
  if (tuned) {
    h->item_rows = desc->item_rows;
    h->item_cols = desc->item_cols;
    h->share_lanes = desc->share_lanes == PL_TUNE_RULE ? -1 : (desc->share_lanes == PL_TUNE_ALWAYS ? 1 : 0);
    h->row_items = desc->row_items == PL_TUNE_RULE ? -1 : (desc->row_items == PL_TUNE_ALWAYS ? 1 : 0);
  }
  // filter rows as the dot-product operand (w0, w1, w2, 0)
  std::vector<uint32_t> wpack(static_cast<size_t>(desc->channels) * 4, 0u);
  for (int c = 0; c < desc->channels; ++c)
    for (int r = 0; r < 3; ++r) {
      const int8_t* w = desc->weights + (static_cast<size_t>(c) * 3 + r) * 3;
      wpack[static_cast<size_t>(c) * 4 + r] = static_cast<uint32_t>(static_cast<uint8_t>(w[0])) | static_cast<uint32_t>(static_cast<uint8_t>(w[1])) << 8 | static_cast<uint32_t>(static_cast<uint8_t>(w[2])) << 16;
    }
  std::vector<float> bias(desc->channels, 0.0f);
  if (desc->bias) std::memcpy(bias.data(), desc->bias, sizeof(float) * desc->channels);
  if ((e = h->wpack.Upload(wpack.data(), wpack.size() * 4)) != hipSuccess) return FailHip(e, "uploading the filters");
  if ((e = h->scale.Upload(desc->scale, sizeof(float) * desc->channels)) != hipSuccess) return FailHip(e, "uploading the scales");
  if ((e = h->bias.Upload(bias.data(), sizeof(float) * desc->channels)) != hipSuccess) return FailHip(e, "uploading the biases");
  *out_handle = h.release();
  return PL_OK;
}

int pl_dwconv3x3_run(pl_dwconv_handle* h, const int8_t* x_dev, void* out_dev, int32_t batch, int32_t height, int32_t width, void* stream) {
  if (!h) return Fail(PL_ERR_BAD_ARG, "null handle");
  if (batch < 0 || height <= 0 || width <= 0) return Fail(PL_ERR_BAD_ARG, "bad batch or input size");
  const int oh = (height + 2 * h->pad - 3) / h->stride + 1, ow = (width + 2 * h->pad - 3) / h->stride + 1;
  if (height + 2 * h->pad < 3 || width + 2 * h->pad < 3) return Fail(PL_ERR_BAD_ARG, "the input is smaller than the filter");
  if (batch == 0) return PL_OK;
  if (!x_dev || !out_dev) return Fail(PL_ERR_BAD_ARG, "null device pointer");
  int cur_dev = -1;
  if (hipGetDevice(&cur_dev) != hipSuccess || cur_dev != h->device) return Fail(PL_ERR_BAD_ARG, "the handle belongs to device %d, the current device is %d", h->device, cur_dev);
  const int64_t planes = static_cast<int64_t>(batch) * h->channels;
  if (planes > 0x7fffffffll || planes * height * width >= (1ll << 40)) return Fail(PL_ERR_UNSUPPORTED, "tensor too large");
  if (static_cast<int64_t>((oh + 1) / 2) * ((ow + 3) / 4) >= (1ll << 24)) return Fail(PL_ERR_UNSUPPORTED, "output planes of 2^24 and more items of two rows by four columns are not supported");
  pl::DwConvParams p{};
  p.x = x_dev;
  p.out = out_dev;
  p.wpack = static_cast<const uint32_t*>(h->wpack.ptr);
  p.scale = static_cast<const float*>(h->scale.ptr);
  p.bias = static_cast<const float*>(h->bias.ptr);
  p.channels = h->channels;
  p.h = height;
  p.w = width;
  p.oh = oh;
  p.ow = ow;
  p.pad = h->pad;
  p.planes = static_cast<uint32_t>(planes);
  p.in_bytes = planes * height * width;
  p.act = h->act;
  p.item_rows = h->item_rows;
  p.item_cols = h->item_cols;
  p.share_lanes = h->share_lanes;
  p.row_items = h->row_items;
  const hipError_t e = pl::LaunchDwConv3x3(h->stride, h->kind == PL_KIND_INT8_INT8 ? pl::kOutI8 : pl::kOutF32, p, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? PL_OK : FailHip(e, "depthwise convolution launch");
}

void pl_dwconv3x3_destroy(pl_dwconv_handle* h) { delete h; }

// ---- pointwise + depthwise in one launch -----------------------------------
namespace {
// nullptr when the pair can run as one launch, else the reason
const char* FusedPairProblem(const pl_sparse_conv_handle* c, const pl_dwconv_handle* d, int height, int width) {
  if (c->kind != PL_KIND_INT8_INT8 || d->kind != PL_KIND_INT8_INT8) return "both layers must be int8 -> int8";
  if (c->device != d->device) return "the handles belong to different devices";
  if (c->wtiles_rows.ptr == nullptr) return "the pointwise handle holds no row tiles (oc % 128 == 0 and ic = 128, 256 or 512 are needed)";
  if (!c->auto_int8 && c->algo != PL_ALGO_IMAGE_MFMA) return "the pointwise handle is tied to another algorithm";
  if (c->image_kernel != 0 && c->image_kernel != 3) return "the pointwise handle is tied to another image kernel";
  if (d->channels != c->oc) return "the depthwise layer must have as many channels as the pointwise layer has output channels";
  if (!pl::ImageRowsDwFits(c->oc, c->ic, height * width, height, width, d->pad, d->stride)) return "needs 14 x 14 maps, depthwise padding 1 and stride 1 or 2";
  return nullptr;
}
}  // namespace

int pl_sparse_conv_dwconv3x3_fits(const pl_sparse_conv_handle* conv, const pl_dwconv_handle* dw, int32_t height, int32_t width) {
  if (!conv || !dw || height <= 0 || width <= 0) return 0;
  return FusedPairProblem(conv, dw, height, width) == nullptr ? 1 : 0;
}

int pl_sparse_conv_dwconv3x3_pays(const pl_sparse_conv_handle* conv, const pl_dwconv_handle* dw, int32_t batch, int32_t height, int32_t width) {
  if (!pl_sparse_conv_dwconv3x3_fits(conv, dw, height, width) || batch <= 0) return 0;
  // Measured on 512 -> 512 @14x14 (us, two launches against one, at 1 / 16 / 32 / 48 / 64 images): stride 2: 9.3 / 8.2,
  // 9.8 / 8.4, 10.3 / 8.5, 11.0 / 8.6, 11.9 / 8.8; stride 1: 9.6 / 10.7, 10.4 / 11.1, 11.4 / 11.3, 12.7 / 11.5, 13.8 / 11.8.
  // The one launch does the depthwise work of 128 planes on the CU that made them, whatever the batch; the
  // depthwise kernel spreads a small batch over the chip.
  if (dw->stride == 2) return 1;
  const int64_t workgroups = static_cast<int64_t>(batch) * (conv->oc / 128);
  const int cus = std::max(1, conv->wg_slots_default / 2);
  return workgroups * 2 >= static_cast<int64_t>(cus) ? 1 : 0;
}

int pl_sparse_conv_dwconv3x3_run(pl_sparse_conv_handle* conv, pl_dwconv_handle* dw, const void* x_dev, void* out_dev, int32_t batch, int32_t height, int32_t width, void* stream) {
  if (!conv || !dw) return Fail(PL_ERR_BAD_ARG, "null handle");
  if (batch < 0 || height <= 0 || width <= 0) return Fail(PL_ERR_BAD_ARG, "bad batch or input size");
  if (const char* why = FusedPairProblem(conv, dw, height, width)) return Fail(PL_ERR_UNSUPPORTED, "pointwise + depthwise in one launch: %s", why);
  if (batch == 0) return PL_OK;
  if (!x_dev || !out_dev) return Fail(PL_ERR_BAD_ARG, "null device pointer");
  int cur_dev = -1;
  if (hipGetDevice(&cur_dev) != hipSuccess || cur_dev != conv->device) return Fail(PL_ERR_BAD_ARG, "the handles belong to device %d, the current device is %d", conv->device, cur_dev);
  if (static_cast<int64_t>(batch) * conv->oc > 0x7fffffffll) return Fail(PL_ERR_UNSUPPORTED, "tensor too large");
  if (reinterpret_cast<uintptr_t>(x_dev) % 4 != 0 || reinterpret_cast<uintptr_t>(out_dev) % 4 != 0) return Fail(PL_ERR_UNSUPPORTED, "pointwise + depthwise in one launch needs 4-byte aligned tensors");
  pl::ImageMfmaParams p{};
  p.x = static_cast<const int8_t*>(x_dev);
  p.out = nullptr;
  p.wtiles = conv->wtiles_rows.ptr;
  p.scale = static_cast<const float*>(conv->scale.ptr);
  p.bias = static_cast<const float*>(conv->bias.ptr);
  p.M = conv->oc;
  p.K = conv->ic;
  p.hw = height * width;
  p.batch = batch;
  p.act = conv->act;
  pl::DwConvParams d{};
  d.x = nullptr;
  d.out = out_dev;
  d.wpack = static_cast<const uint32_t*>(dw->wpack.ptr);
  d.scale = static_cast<const float*>(dw->scale.ptr);
  d.bias = static_cast<const float*>(dw->bias.ptr);
  d.channels = dw->channels;
  d.h = height;
  d.w = width;
  d.oh = (height + 2 * dw->pad - 3) / dw->stride + 1;
  d.ow = (width + 2 * dw->pad - 3) / dw->stride + 1;
  d.pad = dw->pad;
  d.planes = static_cast<uint32_t>(static_cast<int64_t>(batch) * dw->channels);
  d.in_bytes = static_cast<int64_t>(d.planes) * height * width;
  d.act = dw->act;
  const hipError_t e = pl::LaunchImageRowsDw(p, d, dw->stride, static_cast<hipStream_t>(stream));
  return e == hipSuccess ? PL_OK : FailHip(e, "pointwise + depthwise launch");
}

}  // extern "C"
