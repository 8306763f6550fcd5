// Launch geometry of the copy-shaped kernels (copy, broadcast, array converters, pack / unpack) and the host's choices
// for a reduce (where its vectors start, whether its phased form pays): plain arithmetic, kept apart from the kernels
// so that it can be compiled and tested without a GPU.
//
// These kernels give every lane one group of elements (one 16-byte vector, or the 4 or 8 elements that make one) and
// every block one tile of kGeomBlock groups.  HIP refuses a launch whose gridDim.x * blockDim.x reaches 2^32, i.e. more
// than 2^24 - 1 blocks of 256 lanes: 64 GiB of copy output.  Larger work is cut into several launches, each over its
// own contiguous run of tiles.
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define MI_GEOM_HD __host__ __device__
#else
#define MI_GEOM_HD
#endif

namespace mi {

constexpr uint32_t kGeomBlock = 256;

// blocks of `block` lanes one launch may have
inline uint64_t hip_block_limit(uint32_t block) {
    return ((1ull << 32) / block) - 1;
}

// `count` elements written to an array whose first byte is at address `out_addr`: `head` elements up to the array's
// first 16-byte boundary, then `ngroup` groups of `per` elements (one group per lane), then `tail` elements.  The head
// and tail elements (fewer than a group each) are handled one per lane by block 0 of a launch.
struct LaneWork {
    uint32_t head;
    uint64_t ngroup;
    uint32_t tail;
};
inline LaneWork lane_work(uint64_t out_addr, uint32_t out_elem_bytes, uint64_t count, uint32_t per, uint32_t boundary = 16) {
    LaneWork w;
    const uint64_t mis = out_addr & (boundary - 1);     // boundary: 16, or 128 to start the vectors on a line of the output
    uint64_t head = ((boundary - mis) & (boundary - 1)) / out_elem_bytes;
    if (head > count) head = count;
    w.head = (uint32_t)head;
    w.ngroup = (count - head) / per;
    w.tail = (uint32_t)(count - head - w.ngroup * per);
    return w;
}

// One launch of the work: groups [group0, group0 + ngroup) by `grid` blocks; the first launch also takes the head
// elements and the last one the tail elements.  Pointers are advanced by the caller so that the kernel sees a piece
// as if it were the whole job (a piece other than the first has no head).
struct LaunchPiece {
    uint64_t group0, ngroup;
    uint32_t head, tail, grid;
};
inline uint64_t num_launches(const LaneWork& w, uint32_t block, uint64_t limit) {
    const uint64_t tiles = (w.ngroup + block - 1) / block;
    return tiles ? (tiles + limit - 1) / limit : 1;
}
inline LaunchPiece launch_piece(const LaneWork& w, uint32_t block, uint64_t limit, uint64_t i) {
    const uint64_t tiles = (w.ngroup + block - 1) / block;
    const uint64_t n = num_launches(w, block, limit);
    const uint64_t t0 = i * limit, t1 = (t0 + limit < tiles) ? t0 + limit : tiles;
    LaunchPiece p;
    p.group0 = t0 * block;
    const uint64_t end = (t1 * block < w.ngroup) ? t1 * block : w.ngroup;
    p.ngroup = end > p.group0 ? end - p.group0 : 0;
    p.head = i == 0 ? w.head : 0;
    p.tail = i == n - 1 ? w.tail : 0;
    p.grid = (uint32_t)(t1 > t0 ? t1 - t0 : 1);
    return p;
}

// One buffer to m buffers.  The source's tiles are taken in sections of `sect_tiles` tiles; within a section, all of
// its tiles go to destination 0, then all of them to destination 1, and so on: `per` = sect_tiles * m blocks per
// section.  A launch takes whole sections.
struct BcastShape {
    uint32_t head, tail;
    uint64_t nvec;
    uint32_t sect_tiles;    // a multiple of 8, so that a tile is always handled on the same XCD
    uint64_t sects;
};
inline BcastShape bcast_shape(uint64_t dst0_addr, uint64_t bytes, uint32_t max_sect_tiles, uint32_t boundary = 16) {
    const LaneWork w = lane_work(dst0_addr, 1, bytes, 16, boundary);
    BcastShape b;
    b.head = w.head;
    b.nvec = w.ngroup;
    b.tail = w.tail;
    uint64_t tiles = (b.nvec + kGeomBlock - 1) / kGeomBlock;
    if (tiles == 0) tiles = 1;
    b.sect_tiles = tiles < max_sect_tiles ? (uint32_t)((tiles + 7) & ~7ull) : max_sect_tiles;
    b.sects = (tiles + b.sect_tiles - 1) / b.sect_tiles;
    return b;
}
struct BcastPiece {
    uint64_t vec0, nvec;    // vectors [vec0, vec0 + nvec) of the source
    uint32_t head, tail, grid;
};
inline uint64_t bcast_sects_per_launch(const BcastShape& b, int m, uint64_t limit) {
    const uint64_t per = (uint64_t)b.sect_tiles * (uint64_t)m;
    const uint64_t s = limit / per;
    return s ? s : 1;
}
inline uint64_t bcast_num_launches(const BcastShape& b, int m, uint64_t limit) {
    const uint64_t s = bcast_sects_per_launch(b, m, limit);
    return (b.sects + s - 1) / s;
}
inline BcastPiece bcast_piece(const BcastShape& b, int m, uint64_t limit, uint64_t i) {
    const uint64_t s = bcast_sects_per_launch(b, m, limit), n = bcast_num_launches(b, m, limit);
    const uint64_t s0 = i * s, s1 = (s0 + s < b.sects) ? s0 + s : b.sects;
    BcastPiece p;
    p.vec0 = s0 * b.sect_tiles * kGeomBlock;
    const uint64_t end = (s1 * b.sect_tiles * kGeomBlock < b.nvec) ? s1 * b.sect_tiles * kGeomBlock : b.nvec;
    p.nvec = end > p.vec0 ? end - p.vec0 : 0;
    p.head = i == 0 ? b.head : 0;
    p.tail = i == n - 1 ? b.tail : 0;
    p.grid = (uint32_t)((s1 - s0) * b.sect_tiles * (uint64_t)m);
    return p;
}
// which destination and which vector of the piece a lane of block `blk` handles
struct BcastLane {
    uint32_t dst;
    uint64_t vec;
};
MI_GEOM_HD inline BcastLane bcast_lane(uint32_t blk, uint32_t tid, uint32_t sect_tiles, uint32_t m) {
    const uint32_t per = sect_tiles * m;
    const uint32_t sect = blk / per, r = blk - sect * per;
    const uint32_t k = r / sect_tiles, t = r - k * sect_tiles;
    BcastLane l;
    l.dst = k;
    l.vec = ((uint64_t)sect * sect_tiles + t) * kGeomBlock + tid;
    return l;
}

// ---- where the 16-byte vectors of a reduce start -----------------------------------------------------------------
// The vectors start on a 16-byte boundary of one of the buffers; every buffer that disagrees with it is read or
// written as loose vectors, and what that costs depends on which they are.  Measured with the phased kernel on
// 8 x 1 GiB bf16 (7.14 TB/s with everything aligned): seven inputs 4 bytes off the grid 7.00 (-2 %: a loose read on a
// 4-byte boundary is nearly free), eight inputs 2 bytes off 5.66 (-21 %: off the 4-byte boundary a loose read is
// dear), the output alone off the grid, by 4 or by 6 bytes, 6.67-6.80 (-5 to -7 %).  So every candidate boundary is
// priced -- 1 per input that is off it by a multiple of 4 bytes, 8 per input off it otherwise, 16 per output off it --
// and the cheapest wins, the first destination's among equals.  (A plain majority, the rule before, put the grid on
// seven peers 4 bytes off and paid for a loose output: 6.67 against 7.00.)
// With the kernels' realignment in registers (reduce_kernels.hpp, load_vectors) an input off the 4-byte boundary is
// read on that boundary like one that is a multiple of 4 bytes off, plus one more load per wave and a few ALU
// instructions per vector.  Measured on the same 8 x 1 GiB bf16 (7.13 TB/s aligned): seven peers realigned 6.68 (-0.9 %
// per input), eight inputs realigned 6.24 (-1.6 % per input), against -2.6 % per input for loose reads off the 4-byte
// boundary (four of eight inputs: 6.39 loose, 6.90 realigned) and -6.4 % for a loose output: about half the price.
constexpr unsigned kRealignedReadPrice = 4;
inline unsigned loose_read_price(unsigned off, bool realign) {
    return (off & 15u) == 0 ? 0u : (off & 3u) == 0 ? 1u : realign ? kRealignedReadPrice : 8u;
}
constexpr unsigned kLooseWritePrice = 16;
inline unsigned grid_price(unsigned c, const unsigned* in_mis, int n, const unsigned* out_mis, int m, bool realign = false) {
    unsigned p = 0;
    for (int j = 0; j < n; j++) p += loose_read_price(in_mis[j] - c, realign);
    for (int k = 0; k < m; k++) p += ((out_mis[k] - c) & 15u) == 0 ? 0u : kLooseWritePrice;
    return p;
}
// in_mis / out_mis: the buffers' addresses modulo 16; realign: inputs off a 4-byte boundary are realigned in registers
// by the kernel; returns the address modulo 16 at which the vectors start
inline unsigned vector_grid(const unsigned* in_mis, int n, const unsigned* out_mis, int m, bool realign = false) {
    unsigned mis = out_mis[0] & 15u, best = grid_price(mis, in_mis, n, out_mis, m, realign);
    for (int k = 1; k < m; k++) {
        const unsigned p = grid_price(out_mis[k], in_mis, n, out_mis, m, realign);
        if (p < best) { best = p; mis = out_mis[k] & 15u; }
    }
    for (int j = 0; j < n; j++) {
        const unsigned p = grid_price(in_mis[j], in_mis, n, out_mis, m, realign);
        if (p < best) { best = p; mis = in_mis[j] & 15u; }
    }
    return mis;
}

// ---- which 128-byte line the vectors start on ----------------------------------------------------------------------
// Loads and stores here stream past the caches (non-temporal), so a 128-byte line that two waves share -- the ends of
// every wave's 1 KiB when a buffer is 16-byte but not 128-byte aligned -- is often fetched twice, and written in two
// parts.  Measured with the phased kernel on 8 x 512 MiB bf16 (7.09 TB/s with everything on lines): seven peers 16 or
// 64 bytes off 6.94 (-0.3 % per input; 128 bytes off costs nothing), the output alone 16 bytes off 6.80 (-4 %),
// everything 16 bytes off 6.66; own input and output 64 bytes off 7.04 (a store of 64 whole bytes is cheap wherever it
// lies in its line).  So the head is lengthened by whole vectors until the buffers that matter most start on a line:
// 13 per output that is off the 64-byte boundary, 1 per output or input that is off the line otherwise, counted over
// the buffers that agree with the vectors' 16-byte boundary (the others are loose anyway); among equals the head stays
// as it is, then the first destination's line wins.  With that rule the same cases measure 6.97 (peers off), 6.96
// (output off), 7.10 (everything 16 bytes, or 2 bytes, off).
// in_addr / out_addr: addresses modulo 128; mis: vector_grid's answer.  Returns the bytes before the first vector
// (a multiple of 16 on top of what reaches the 16-byte boundary; at most 127).
constexpr unsigned kLineBytes = 128;
constexpr unsigned kLineWritePrice = 13;
inline unsigned line_price(unsigned start, const unsigned* in_addr, int n, const unsigned* out_addr, int m) {
    unsigned p = 0;
    for (int j = 0; j < n; j++)
        if (((in_addr[j] + start) & 15u) == 0 && ((in_addr[j] + start) & (kLineBytes - 1))) p += 1;
    for (int k = 0; k < m; k++)
        if (((out_addr[k] + start) & 15u) == 0 && ((out_addr[k] + start) & (kLineBytes - 1)))
            p += ((out_addr[k] + start) & 63u) ? kLineWritePrice : 1u;
    return p;
}
inline unsigned vector_start(const unsigned* in_addr, int n, const unsigned* out_addr, int m, unsigned mis, bool lines) {
    const unsigned h0 = (16u - mis) & 15u;
    if (!lines) return h0;
    unsigned best_start = h0, best = line_price(h0, in_addr, n, out_addr, m);
    auto consider = [&](unsigned addr) {
        if ((addr + h0) & 15u) return;
        const unsigned start = h0 + ((kLineBytes - ((addr + h0) & (kLineBytes - 1))) & (kLineBytes - 1));
        const unsigned p = line_price(start, in_addr, n, out_addr, m);
        if (p < best) {
            best = p;
            best_start = start;
        }
    };
    for (int k = 0; k < m; k++) consider(out_addr[k]);
    for (int j = 0; j < n; j++) consider(in_addr[j]);
    return best_start;
}

// ---- the pace of a phased reduce's write phase --------------------------------------------------------------------------
// The kernel lets group i of four stores per lane out at the phase's start + i * pace: `bytes_per_group` is what the
// whole grid stores in one group, `rate_gbps` the rate in GB/s the groups are let out at, `clock_khz` the rate of the
// device's wall clock.  Returns the pace in 1/16 clock ticks (0: unpaced).
inline uint32_t write_pace_ticks16(uint64_t bytes_per_group, double rate_gbps, int clock_khz) {
    if (rate_gbps <= 0 || clock_khz <= 0) return 0;
    const double ticks16 = (double)bytes_per_group / (rate_gbps * 1e9) * (double)clock_khz * 1e3 * 16.0 + 0.5;
    return ticks16 >= 4294967295.0 ? 4294967295u : (uint32_t)ticks16;
}

// ---- when the phased form of a reduce pays -----------------------------------------------------------------------
// A phase costs a fixed few microseconds on top of its traffic, so what counts is how full the phases are:
// fill = result vectors / (phases x what one phase holds).  Measured against the streaming kernels (fp32 sum, one
// destination, rotating buffer sets): with 2 inputs the phased form wins at fill 0.97 (+1 to +8 % from 256 MiB of
// traffic up) and loses at 0.73; with 3 it wins at 0.73 (+2-3 %) and loses at 0.55; with 4 it wins at 0.58 and loses at
// 0.44; with 8 it wins from 0.32 (+3 %) and is even at 0.24: about 2 / n.
inline bool phases_full_enough(uint64_t nvec, uint64_t vectors_per_phase, int n_inputs) {
    if (nvec == 0 || vectors_per_phase == 0 || n_inputs < 1) return false;
    const uint64_t phases = (nvec + vectors_per_phase - 1) / vectors_per_phase;
    const double fill = (double)nvec / (double)(phases * vectors_per_phase);
    const double need = 2.0 / n_inputs < 0.9 ? 2.0 / n_inputs : 0.9;
    return fill >= need;
}

// How many groups of four result vectors per lane a launch of the phased reduce keeps in registers: the usual
// `groups`, or one more when that takes a whole phase off a launch of at most kPhaseWiderUpTo phases (`lanes` lanes
// on the chip, lds_vectors more vectors per lane in LDS).  A phase costs a fixed 5-9 us, so 96 MiB of results in one
// phase instead of 88 MiB and a sliver measure 74.8 against 81.0 us with 4 fp32 inputs and 134.2 against 139.9 us
// with 8 bfloat16 ones; 192 MiB in two phases instead of three 148.1 against 153.6 and 266.5 against 269.5; 384 MiB in
// four instead of five 293.5 against 297.7 and 525 against 533.  With the phase count unchanged the wider phase measures 0.5-1.7 % slower,
// and from seven phases on one phase less no longer shows (1 GiB: 11 against 12 phases, 2 GB: 20 against 22, both
// within 0.2 %): the usual width stays there.
constexpr uint64_t kPhaseWiderUpTo = 6;
inline int phase_reg_groups(uint64_t nvec, uint64_t lanes, int groups, int lds_vectors) {
    const uint64_t usual = lanes * (uint64_t)(4 * groups + lds_vectors), wider = lanes * (uint64_t)(4 * (groups + 1) + lds_vectors);
    if (nvec == 0 || usual == 0) return groups;
    const uint64_t p_usual = (nvec + usual - 1) / usual, p_wider = (nvec + wider - 1) / wider;
    return (p_wider < p_usual && p_usual <= kPhaseWiderUpTo) ? groups + 1 : groups;
}

// The same question for a batch of jobs whose vectors are laid end to end in tiles of tile_vectors vectors, every job
// padded to whole tiles: `vectors` result vectors in `tiles` tiles, tiles_per_phase tiles to a phase.  The padding
// counts as empty space like the unused end of the last phase.
inline bool batch_phases_full_enough(uint64_t vectors, uint64_t tiles, uint64_t tiles_per_phase, uint64_t tile_vectors, int n_inputs) {
    if (vectors == 0 || tiles == 0 || tiles_per_phase == 0 || n_inputs < 1) return false;
    const uint64_t phases = (tiles + tiles_per_phase - 1) / tiles_per_phase;
    const double fill = (double)vectors / (double)(phases * tiles_per_phase * tile_vectors);
    const double need = 2.0 / n_inputs < 0.9 ? 2.0 / n_inputs : 0.9;
    return fill >= need;
}

// ---- pack / unpack: the 4 KiB quarters of one tensor, cut where the destination crosses a 128-byte line -------------
// Quarter q of a tensor of `total` bytes whose destination starts at address dst_addr covers bytes [lo, lo + n) of
// the tensor: quarter 0 ends at the destination's first line boundary at or before 4 KiB, every further quarter starts
// on a line boundary and is 4 KiB, the last one takes what is left (n <= 4 KiB + 127).  n == 0: no such quarter.
constexpr uint32_t kCopyQuarter = 4096;
constexpr uint32_t kCopyLine = 128;
struct CopyQuarter {
    uint64_t lo;
    uint32_t n;
};
MI_GEOM_HD inline CopyQuarter copy_quarter(uint64_t total, uint64_t dst_addr, uint64_t q) {
    const uint64_t nq = (total + kCopyQuarter - 1) / kCopyQuarter;
    CopyQuarter r = { 0, 0 };
    if (q >= nq) return r;
    const uint64_t lack = (0 - dst_addr) & (kCopyLine - 1);     // bytes to the destination's first line boundary
    const uint64_t back = lack ? kCopyLine - lack : 0;
    r.lo = q ? q * kCopyQuarter - back : 0;
    const uint64_t hi = (q + 1 == nq) ? total : (q + 1) * kCopyQuarter - back;
    r.n = (uint32_t)(hi - r.lo);
    return r;
}

}  // namespace mi
