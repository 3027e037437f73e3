// The attention kernels' view of a window whose position lives in a device word: which cache positions a block may read.
// The host cannot check a position it does not know, so the kernels bound every index by the cache's capacity here; a
// window that does not fit is reported through an error bit and computed over the cells that exist. Plain functions of
// integers, compiled for the device and (by the bounds test) for the host.
#pragma once

#if defined(__HIPCC__)
#define FNX_HOST_DEVICE __host__ __device__
#else
#define FNX_HOST_DEVICE
#endif

namespace fnx {

constexpr int AT_SPLIT = 512;   // positions a block of the first pass covers
constexpr int AT_CH = 32;       // positions a chunk (one trip of a block's loop)
constexpr int AT_VB = 8;        // positions whose values of a dimension lie together in the V cache: [position / 8][kv head][dim][position % 8]

FNX_HOST_DEVICE inline int att_min(int a, int b) { return a < b ? a : b; }
FNX_HOST_DEVICE inline int att_max(int a, int b) { return a > b ? a : b; }
FNX_HOST_DEVICE inline int attn_splits(int max_ctx) { return (max_ctx + AT_SPLIT - 1) / AT_SPLIT; }

struct AttWindow {
    int pos0;      // the first row's position, not below 0 and not past the cache's last cell
    int ctx_max;   // the last row sees positions [0, ctx_max): 1 .. max_ctx
};
// T rows at positions pos0_raw .. pos0_raw + T - 1 of a cache of max_ctx >= 1 cells
FNX_HOST_DEVICE inline AttWindow att_window(int pos0_raw, int T, int max_ctx) {
    const int pos0 = att_min(att_max(pos0_raw, 0), max_ctx - 1);
    return AttWindow{pos0, att_min(pos0 + att_max(T, 1), max_ctx)};
}
FNX_HOST_DEVICE inline bool att_window_fits(int pos0_raw, int T, int max_ctx) { return pos0_raw >= 0 && T >= 1 && pos0_raw <= max_ctx - T; }
// row qt of the window sees positions [0, this)
FNX_HOST_DEVICE inline int att_ctx_q(const AttWindow& w, int qt) { return att_min(w.pos0 + qt + 1, w.ctx_max); }
// A window of few queries (those of a kv head fit one block of the first pass: AT_HALF_QUERIES) leaves the blocks of the
// grid's second layer without queries; they take the second half of their split instead, so that such a window - a decode
// round's, most of the time - is spread over as many blocks as a full one. Part (s, z) of the first pass covers positions
// [begin, end) (empty when begin >= end) and is part number att_part_index of its query; halves: the window is such a one.
constexpr int AT_HALF_QUERIES = 64;
FNX_HOST_DEVICE inline bool att_halves(int nquery) { return nquery <= AT_HALF_QUERIES; }
FNX_HOST_DEVICE inline int att_part_begin(int s, int z, bool halves) { return s * AT_SPLIT + (halves ? z * (AT_SPLIT / 2) : 0); }
FNX_HOST_DEVICE inline int att_part_end(const AttWindow& w, int s, int z, bool halves) {
    return att_min(w.ctx_max, att_part_begin(s, z, halves) + (halves ? AT_SPLIT / 2 : AT_SPLIT));
}
FNX_HOST_DEVICE inline int att_part_index(int s, int z, bool halves) { return halves ? 2 * s + z : s; }
// the parts a query's row of the scratch area has room for, and the parts that the first pass wrote with data (the second
// pass reads these)
FNX_HOST_DEVICE inline int att_part_slots(int nsplit) { return 2 * nsplit; }
// the parts between one query's first and the next one's in the scratch area: a full window's lie as closely as they did
// without the halves (the window's mode is the same for both passes: they read the same device words)
FNX_HOST_DEVICE inline int att_part_stride(int nsplit, bool halves) { return halves ? 2 * nsplit : nsplit; }
FNX_HOST_DEVICE inline int att_live_parts(const AttWindow& w, int nsplit, bool halves) {
    const int len = halves ? AT_SPLIT / 2 : AT_SPLIT;
    return att_min(halves ? 2 * nsplit : nsplit, (w.ctx_max + len - 1) / len);
}
// the K row and the V block (of AT_VB positions) that a fetch of chunk c0 reads for its row r (0 .. AT_CH - 1) and block b
// (0 .. AT_CH / AT_VB - 1): clamped inside the window's rows
FNX_HOST_DEVICE inline int att_fetch_row(const AttWindow& w, int c0, int r) { return att_min(c0 + r, w.ctx_max - 1); }
FNX_HOST_DEVICE inline int att_fetch_vblock(const AttWindow& w, int c0, int b) { return att_min(c0 / AT_VB + b, (w.ctx_max - 1) / AT_VB); }

}  // namespace fnx
