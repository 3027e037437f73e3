// How the one-launch verify window (k_moe_window.h) cuts a window's work over the grid: which row a block belongs to, its
// router rows, its run of gate|up items, its units of the down matrices, and how many blocks each of a row's two
// hand-overs waits for. Plain functions of integers, compiled for the device and (by the plan test) for the host, so
// that every count a block waits for can be checked against the blocks that arrive without running a kernel.
#pragma once

#if defined(__HIPCC__)
#define FNX_HOST_DEVICE __host__ __device__
#else
#define FNX_HOST_DEVICE
#endif

namespace fnx {

constexpr int WN_WAVES = 16;   // waves a block

struct WinPlan {
    int Tl;        // rows of the window that count
    int G;         // blocks a row, a power of two; block b belongs to row b / G and is the row's block b % G
    int nk, k0;    // matrices a row's gate|up items walk (the shared expert's if k0 == 0, then the picks'), the first one
    int qpp;       // blocks of 32 h values a pair
    int per_row;   // gate|up items a row: qpp * nk, numbered (block of 32, matrix)
    int ipb;       // items a block: block g takes items [g * ipb, min(per_row, (g + 1) * ipb))
    int nbi;       // blocks of a row that have items: the count the row's h hand-over waits for
    int rpb;       // router rows a block: block g takes rows [g * rpb, min(nexp, (g + 1) * rpb))
    int upb;       // units of a down matrix a block: block g takes units [g * upb, (g + 1) * upb)
    int R;         // of them a wave and trip; wave w < dwaves takes units g * upb + w * R .. + R - 1
    int dwaves;    // waves with units
};

FNX_HOST_DEVICE inline int win_pow2_floor(int v) {
    int p = 1;
    while (2 * p <= v) p *= 2;
    return p;
}
// nb: blocks of the grid; Tl >= 1 rows that count; nexp experts, topk picks a row; shared: the shared expert's matrices are
// this launch's; ff: expert width (a multiple of 256: the down matrices have 2048 rows of ff columns = ff units of 64 sub-blocks)
FNX_HOST_DEVICE inline WinPlan win_plan(int nb, int Tl, int nexp, int topk, bool shared, int ff) {
    WinPlan p;
    p.Tl = Tl;
    p.G = win_pow2_floor(nb / Tl);
    if (p.G > ff) p.G = ff;   // at least one unit of the down matrices a block (ff is a power of two times 256)
    p.k0 = shared ? 0 : 1;
    p.nk = topk + 1 - p.k0;
    p.qpp = ff / 32;
    p.per_row = p.qpp * p.nk;
    p.ipb = (p.per_row + p.G - 1) / p.G;
    p.nbi = (p.per_row + p.ipb - 1) / p.ipb;
    p.rpb = (nexp + p.G - 1) / p.G;
    p.upb = ff / p.G;
    p.dwaves = p.upb < WN_WAVES ? p.upb : WN_WAVES;
    p.R = p.upb / p.dwaves;
    return p;
}
// the most units a wave can hold a trip for rows of SBR sub-blocks (the registers of a block of sixteen waves)
FNX_HOST_DEVICE inline int win_rmax(int sbr) { return sbr / 8; }

}  // namespace fnx
