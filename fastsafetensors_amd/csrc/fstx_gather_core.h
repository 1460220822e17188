// SPDX-License-Identifier: Apache-2.0
//
// Lane logic of the gather kernel, written against a small memory interface so that the very
// same code runs per lane on the GPU (fstx_kernels.hip) and per simulated lane on the CPU,
// where every access is checked against the ranges it may touch (tests/kernel_sim).  No
// wavefront intrinsics in here: a lane depends on nothing but its tile index, its lane index
// and the tables, and everything that is derived from the tile index alone is uniform across
// the wavefront (the compiler keeps it in scalar registers and fetches the tables with scalar
// loads).
//
// The job.  A destination of `rows` rows, `dst_pitch` bytes apart, each holding `row_bytes`
// payload bytes: the segments of `nsrc` sources side by side, source k contributing `seg`
// bytes per row at column `col`, read from `src + row * pitch`.  One source and
// dst_pitch == row_bytes is a rank's block of one tensor (slice extract); several sources are
// the rank's blocks of several tensors joined along an inner dimension.  Nothing has to be
// aligned: not the destination, not the pitches, not the segment lengths.
//
// How it moves.  The destination is cut into the 16-byte vectors of its memory (vector j is
// the 16 aligned bytes at align_down(dst, 16) + 16 j); a lane owns one vector: it finds the
// row and column of the vector's first byte with one 32-bit division, fetches the sixteen
// bytes with ONE load at whatever byte address they have -- the hardware serves 16-byte global
// loads at any alignment, measured at the rate of aligned ones -- and writes them with one
// aligned 16-byte store.  Only the vectors at the seams (a segment ends inside the vector, a
// pitched destination has a gap there, the job begins or ends there) take the slow way: up to
// two loads that stay inside their segments, moved into place and blended in registers, and a
// byte-wise store under a mask when part of the vector is not the job's.  A wavefront thus
// reads about 1 KiB and writes 1 KiB of contiguous memory whatever the shape; no LDS, no
// barrier, one pass.
#ifndef FSTX_GATHER_CORE_H
#define FSTX_GATHER_CORE_H

#include <stdint.h>

#if defined(__HIPCC__)
#define FSTX_HD __host__ __device__ __forceinline__
#define FSTX_UNROLL _Pragma("unroll")
#else
#define FSTX_HD inline
#define FSTX_UNROLL
#endif

namespace fstx_gather {

struct Vec16 {
    uint32_t w[4];
};

// 64 bytes: fetched with one wide scalar load.  A job with one source (a slice extract) carries
// it inside, so that no second, dependent load stands before its data loads; the sources of a
// job with several sit in the launch's table.
struct alignas(64) Job {
    char *dst;          // payload byte 0 of row 0, any alignment
    uint32_t dst_pitch; // bytes between destination rows, >= row_bytes
    uint32_t row_bytes; // payload bytes per row = sum of the sources' seg
    uint32_t rows;
    uint16_t more0;     // nsrc > 1: the sources are table[more0 .. more0 + nsrc) of the launch
    uint16_t nsrc;
    uint32_t nvec;      // vectors covering [align_down(dst, 16), last payload byte]
    uint32_t equal_seg; // != 0: every source has this seg, so column c belongs to source c / seg
    const char *src;    // nsrc == 1: first byte of the block in row 0
    uint64_t pitch;     // nsrc == 1: bytes between its rows; nsrc > 1: magic_of(equal_seg), or 0
    uint32_t seg;       // nsrc == 1: bytes per row, >= kMinSeg
    uint32_t flags;     // kByRows | kShort | kLooseRows
    uint64_t pitch_magic; // magic_of(dst_pitch); kByRows: magic_of(vectors per row)
};

// Job::flags
constexpr uint32_t kByRows = 2; // vectors are counted row by row (see vectors_per_row)
constexpr uint32_t kShort = 4;  // some segment is shorter than kShortSeg: a tile may hold more than three
constexpr uint32_t kLooseRows = 8; // with kByRows, one source: a row's vectors begin at the row's own first byte
constexpr uint32_t kShortSeg = 512;

struct alignas(32) Src {
    const char *src; // first byte of the block in row 0
    uint64_t pitch;  // bytes between rows of the source
    uint32_t seg;    // bytes per row, >= kMinSeg
    uint32_t col;    // byte offset of the block within a destination row
    uint64_t pad;
};

constexpr uint32_t kLanes = 64;
constexpr uint32_t kVec = 16;
constexpr uint32_t kTile = kLanes * kVec; // destination bytes per wavefront
constexpr uint32_t kMinSeg = 16;          // a vector then overlaps at most two segments

// Tile order of every job (a tile = the 1 KiB a wavefront writes; the copy kernels use the same
// order).  Workgroups reach the dies of the device round-robin (eight on a whole MI355X: workgroup
// b runs on die b % 8; four, two or one when the device is a partition of it -- the launch says
// how many) and every die has its own L2, so in dispatch order the two
// tiles either side of a shared line would sit on different dies and the line would be fetched
// from HBM twice, or a destination line written in two parts.  The tiles are therefore dealt out
// in chunks of 8 x 256: within a chunk die d takes tiles [256 d, 256 d + 256) one after the
// other, so shared lines are found in that die's L2, while all dies together still sweep one
// 2 MiB window of the job at a time -- what keeps the memory channels evenly loaded and the dies
// in step (one contiguous eighth of the job per die measured up to 10 % slower on jobs of
// 100 MB, and 20 % slower when the eighths alias on the channels).  Jobs in which nothing is
// shared -- everything on cache-line boundaries -- take the same order: it measured 0-2 % faster
// than dispatch order on them too.  The last, partial chunk is dealt out in equal parts.  A job
// takes ceil(n_tiles / dies) * dies workgroups; false = an idle one.  One die: dispatch order.
constexpr uint32_t kMaxDiesLog2 = 3; // eight dies at most; what a launch is told comes from the device (see dies_log2 on the host side)
constexpr uint32_t kRunLog2 = 8;
FSTX_HD bool tile_for_die(uint32_t lb, uint32_t n_tiles, uint32_t dies_log2, uint32_t &tile) {
    const uint32_t dies = 1u << dies_log2, chunk = dies << kRunLog2;
    const uint32_t full = n_tiles & ~(chunk - 1);
    if (lb < full) {
        tile = (lb & ~(chunk - 1)) | ((lb & (dies - 1)) << kRunLog2) | ((lb >> dies_log2) & ((1u << kRunLog2) - 1));
        return true;
    }
    const uint32_t per_die = (n_tiles - full + dies - 1) >> dies_log2;
    const uint32_t l = lb - full, turn = l >> dies_log2;
    tile = full + (l & (dies - 1)) * per_die + turn;
    return turn < per_die && tile < n_tiles;
}

// Division of a 32-bit number by a divisor known on the host, d >= 2: floor(n / d) is the high
// 64 bits of n * magic_of(d) -- exact for every n below 2^32, because the magic exceeds 2^64 / d
// by less than d / 2^64 per unit of n.  Two multiplications instead of the twenty-odd
// instructions of a division, in the part of a wavefront that runs before its first load.
inline uint64_t magic_of(uint64_t d) { return d < 2 ? 0 : ~0ull / d + 1; }
FSTX_HD uint32_t div_magic(uint32_t n, uint64_t magic) {
    const uint64_t lo = (uint64_t)n * (uint32_t)magic, hi = (uint64_t)n * (uint32_t)(magic >> 32);
    return (uint32_t)((hi + (lo >> 32)) >> 32);
}

// bytes [m, m + 16) of the 32 bytes lo:hi, m in 0..15.  Written with 64-bit shifts and two-way
// selects only: a chain of four-way selects over the eight dwords is turned back into an
// indexed array by the compiler, and that array lands in scratch memory.
FSTX_HD Vec16 window(Vec16 lo, Vec16 hi, uint32_t m) {
    const uint64_t p0 = lo.w[0] | (uint64_t)lo.w[1] << 32, p1 = lo.w[2] | (uint64_t)lo.w[3] << 32;
    const uint64_t p2 = hi.w[0] | (uint64_t)hi.w[1] << 32, p3 = hi.w[2] | (uint64_t)hi.w[3] << 32;
    const bool far = m >= 8;
    const uint64_t a0 = far ? p1 : p0, a1 = far ? p2 : p1, a2 = far ? p3 : p2;
    const uint32_t t = 8 * (m & 7); // 0..56 bits
    const uint64_t r0 = (a0 >> t) | ((a1 << 1) << (63 - t));
    const uint64_t r1 = (a1 >> t) | ((a2 << 1) << (63 - t));
    return Vec16{{(uint32_t)r0, (uint32_t)(r0 >> 32), (uint32_t)r1, (uint32_t)(r1 >> 32)}};
}

// bytes [at, at + take) from b, the rest from a
FSTX_HD Vec16 blend(Vec16 a, Vec16 b, uint32_t at, uint32_t take) {
    Vec16 o;
    FSTX_UNROLL
    for (int i = 0; i < 4; ++i) {
        const int lo = (int)at - 4 * i, hi = (int)(at + take) - 4 * i; // byte range within this dword, unclipped
        const uint32_t below = lo <= 0 ? 0u : lo >= 4 ? 0xffffffffu : (1u << (8 * lo)) - 1u;   // bytes before the range
        const uint32_t upto = hi <= 0 ? 0u : hi >= 4 ? 0xffffffffu : (1u << (8 * hi)) - 1u;    // bytes before its end
        const uint32_t m = upto & ~below;
        o.w[i] = (a.w[i] & ~m) | (b.w[i] & m);
    }
    return o;
}

// v moved by d bytes, d in -15..15: out[i] = v[i - d]; bytes that come from outside v are zero
FSTX_HD Vec16 shifted(Vec16 v, int32_t d) {
    const Vec16 zero = {{0, 0, 0, 0}};
    const bool up = d > 0;
    Vec16 lo, hi;
    FSTX_UNROLL
    for (int i = 0; i < 4; ++i) {
        lo.w[i] = up ? 0u : v.w[i];
        hi.w[i] = up ? v.w[i] : 0u;
    }
    (void)zero;
    return window(lo, hi, up ? kVec - (uint32_t)d : (uint32_t)(-d));
}

// a segment as one lane sees it
struct Piece {
    uint32_t col, len;  // its column within a destination row, its bytes
    const char *bytes;  // its first byte in the source, in the lane's row
    const char *lo, *hi; // the source block's readable range: first byte of its first row, one past the last byte of its last row
};

FSTX_HD Piece piece_from(const char *src, uint64_t pitch, uint32_t seg, uint32_t col, uint32_t row, uint32_t rows) {
    return Piece{col, seg, src + (uint64_t)row * pitch, src, src + (uint64_t)(rows - 1) * pitch + seg};
}

// table entry `index`; the index is uniform across the wavefront, so on the GPU these are scalar loads
FSTX_HD Src src_uniform(const Src *more, uint32_t index) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef uint32_t v8u_ __attribute__((ext_vector_type(8)));
    const v8u_ raw = *reinterpret_cast<const v8u_ *>(&more[__builtin_amdgcn_readfirstlane(index)]);
    Src out;
    __builtin_memcpy(&out, &raw, sizeof out);
    return out;
#else
    return more[index];
#endif
}

// the column of table entry `index` alone (uniform index: one scalar dword)
FSTX_HD uint32_t col_uniform(const Src *more, uint32_t index) {
#if defined(__HIP_DEVICE_COMPILE__)
    return *reinterpret_cast<const uint32_t *>(
        reinterpret_cast<const char *>(&more[__builtin_amdgcn_readfirstlane(index)]) + __builtin_offsetof(Src, col));
#else
    return more[index].col;
#endif
}

// which source holds column c of a row (c < row_bytes): the table is read with scalar loads,
// the comparisons are per lane
FSTX_HD uint32_t source_of(const Job &jb, const Src *more, uint32_t c) {
    if (jb.nsrc == 1) return 0;
    if (jb.equal_seg) return div_magic(c, jb.pitch);
    uint32_t k = 0;
    for (uint32_t i = 1; i < jb.nsrc; ++i) k += c >= col_uniform(more, jb.more0 + i) ? 1u : 0u;
    return k;
}

// the first two segments that reach into a tile, worked out once per wavefront with scalar loads
struct Near {
    Piece a, b;
    uint32_t row_a, row_b;
};

// The segment that holds column c of row `row`.  Nearly every lane lies in one of the two
// segments at the start of its tile (always, when no segment is shorter than a tile) and takes
// the description from there; only lanes beyond them look their own up.
template <bool kMulti>
FSTX_HD Piece piece_of(const Job &jb, const Src *more, uint32_t row, uint32_t c, const Near &near) {
    if (!kMulti || jb.nsrc == 1) return piece_from(jb.src, jb.pitch, jb.seg, 0, row, jb.rows);
    if (row == near.row_a && c >= near.a.col && c - near.a.col < near.a.len) return near.a;
    if (row == near.row_b && c >= near.b.col && c - near.b.col < near.b.len) return near.b;
    const Src s = more[jb.more0 + source_of(jb, more, c)]; // per lane
    return piece_from(s.src, s.pitch, s.seg, s.col, row, jb.rows);
}

// A job's vectors are normally the 16-byte vectors of the memory between its first and its last
// byte, gaps of a pitched destination included -- the lanes that land in a gap have nothing to
// do.  When the gaps are a large part of that memory (a narrow column block written into a wide
// tensor) the vectors are counted row by row instead: row r has the vectors that cover its own
// payload, vectors_per_row of them at most, and a vector never holds bytes of two rows (the gap
// is at least a vector wide).
FSTX_HD uint32_t vectors_per_row(uint32_t row_bytes) { return (row_bytes + 2 * (kVec - 1)) / kVec; }
// One source: the vectors of a row are counted from the row's own first byte instead -- sixteen
// bytes at dst_row + 16 v, wherever that is, and a last one that ends with the row (it overlaps
// its neighbour when the row is not a multiple of sixteen bytes and writes the same bytes again).
// Every vector is whole payload: one load and one store of sixteen bytes at their own addresses,
// no partial vector and no byte-wise store anywhere in the job.
FSTX_HD uint32_t loose_vectors_per_row(uint32_t row_bytes) { return (row_bytes + kVec - 1) / kVec; }
inline bool counts_by_rows(uint64_t dst_pitch, uint64_t row_bytes) {
    const uint64_t gap = dst_pitch - row_bytes;
    return gap >= kVec && gap > dst_pitch / 8;
}

// Tiles of short segments (Job::flags & kShort: some segment is under kShortSeg bytes, so a tile
// may hold four of them, or sixty).  No description of the tile is shared: every lane finds row,
// source and offset of its own vector by arithmetic -- two multiply-highs, or a count over the
// sources' columns when their widths differ -- fetches the two table entries it may need (its
// segment's and the following one's) together, then issues its one or two data loads together:
// two waits per wavefront, whatever the number of seams.  Decided once per wavefront: not the
// job's first or last tile (the caller checks), and no lane of the tile in the first row or
// beyond the last but one of its source block, so that a load which reaches up to 15 bytes
// before or behind its segment stays inside the block.  Returns false for a tile, or on a
// pitched destination a lane, that needs the general way.
template <bool kMulti, bool kPitched, class Mem>
FSTX_HD bool gather_lane_short(const Job &jb, const Src *more, uint32_t t_lo, uint32_t lane, Mem &mem) {
    const uint32_t dst_pitch = kPitched ? jb.dst_pitch : jb.row_bytes;
    const uint32_t row_first = div_magic(t_lo, jb.pitch_magic), row_last = div_magic(t_lo + kTile - 1, jb.pitch_magic);
    if (row_first == 0 || row_last + 2 > jb.rows) return false;
    const uint32_t q = t_lo + kVec * lane; // position of the vector's byte 0
    const uint32_t row = div_magic(q, jb.pitch_magic);
    const uint32_t c = q - row * dst_pitch;
    if (kPitched && c >= jb.row_bytes) return false; // in the gap behind a row's payload
    const bool multi = kMulti && jb.nsrc > 1;
    Src s1 = {jb.src, jb.pitch, jb.seg, 0, 0}, s2 = s1;
    uint32_t row2 = row + 1;
    if (multi) {
        const uint32_t k = source_of(jb, more, c);
        const uint32_t k2 = k + 1 < jb.nsrc ? k + 1 : 0u;
        // both entries before either is used
        s1 = mem.table(more, jb.more0 + k);
        s2 = mem.table(more, jb.more0 + k2);
        row2 = k2 ? row : row + 1;
    }
    const uint32_t in1 = c - s1.col;
    const uint32_t rest = s1.seg - in1;   // bytes of the segment from the vector's byte 0 on
    const bool has2 = rest < kVec;        // it ends inside the vector: the following segment begins `rest` bytes in
    if (kPitched && has2 && row2 != row) return false; // continues behind the gap: partly payload
    Vec16 g2 = {{0, 0, 0, 0}};
    const Vec16 g1 = mem.load16_stream(s1.src + (uint64_t)row * s1.pitch + in1);
    if (has2) g2 = mem.load16(s2.src + (uint64_t)row2 * s2.pitch - rest);
    const uint32_t from2 = has2 ? rest : kVec;
    mem.store16(jb.dst + q, blend(g1, g2, from2, kVec - from2));
    return true;
}

// The common tile, decided once per wavefront: not the job's first or last tile, at most three
// segments reach into it, and none of them lies in the first or last row of its source block.
// Then every vector of the tile is whole payload made of at most two of the three segments, no
// load can leave a source block, and a lane needs no division: the three segments are described
// once per wavefront as spans of destination positions [pos, end); a lane picks its span by two
// comparisons, loads the sixteen bytes that belong at its own position (and those of the
// following span when its span ends inside the vector), blends and stores.  Returns false for a
// tile, or on a pitched destination a lane, that needs the general way below.
template <bool kMulti, bool kPitched, class Mem>
FSTX_HD bool gather_lane_inner(const Job &jb, const Src *more, uint32_t tile, uint32_t lane, Mem &mem) {
    // ---- once per wavefront, in scalar registers.  The scalar unit is shared by the four SIMDs
    // of a compute unit and a tile is due every 190 cycles or so at full memory rate, so this
    // part is kept short: no division, no 64-bit arithmetic, no copies.
    if (kPitched && (jb.flags & kByRows)) {
        // vectors counted row by row, one source: a vector that lies inside a row's payload is one load
        // inside that row's segment and one store (pitch_magic divides by the vectors per row here)
        if (kMulti && jb.nsrc > 1) return false;
        const uint32_t j = tile * kLanes + lane;
        if (jb.flags & kLooseRows) {
            if (j >= jb.nvec) return true;
            const uint32_t per = loose_vectors_per_row(jb.row_bytes);
            const uint32_t r = per == 1 ? j : div_magic(j, jb.pitch_magic);
            const uint32_t at = kVec * (j - r * per);
            const uint32_t off = at + kVec <= jb.row_bytes ? at : jb.row_bytes - kVec; // the last one ends with the row
            mem.store16_any(jb.dst + (uint64_t)r * jb.dst_pitch + off, mem.load16_stream(jb.src + (uint64_t)r * jb.pitch + off));
            return true;
        }
        if (j >= jb.nvec) return false;
        const uint32_t per_row = vectors_per_row(jb.row_bytes);
        const uint32_t row = div_magic(j, jb.pitch_magic);
        const uint32_t v = j - row * per_row;
        char *row_dst = jb.dst + (uint64_t)row * jb.dst_pitch;
        const uint32_t row_head = (uint32_t)((uintptr_t)row_dst & (kVec - 1));
        const uint32_t c = kVec * v - row_head; // column of the vector's byte 0 (wraps when the row begins inside vector 0)
        if ((v == 0 && row_head != 0) || c + kVec > jb.row_bytes) return false; // partly payload, or past the row's end
        mem.store16(row_dst + c, mem.load16_stream(jb.src + (uint64_t)row * jb.pitch + c));
        return true;
    }
    const uint32_t n_tiles = (jb.nvec + kLanes - 1) / kLanes;
    if (tile == 0 || tile + 1 >= n_tiles) return false;
    const uint32_t head = (uint32_t)((uintptr_t)jb.dst & (kVec - 1));
    const uint32_t dst_pitch = kPitched ? jb.dst_pitch : jb.row_bytes;
    const uint32_t t_lo = tile * kTile - head; // position of the tile's first byte
    if (jb.flags & kShort) return gather_lane_short<kMulti, kPitched>(jb, more, t_lo, lane, mem);
    uint32_t row = div_magic(t_lo, jb.pitch_magic);
    uint32_t c0 = t_lo - row * dst_pitch;
    if (kPitched && c0 >= jb.row_bytes) { // the tile begins in the gap behind a row's payload
        c0 = 0;
        ++row;
    }
    const bool multi = kMulti && jb.nsrc > 1;
    uint32_t k = multi ? source_of(jb, more, c0) : 0u;
    uint32_t ks[3], rs[3];
    FSTX_UNROLL
    for (int x = 0; x < 3; ++x) {
        ks[x] = k;
        rs[x] = row;
        if (++k == jb.nsrc) {
            k = 0;
            ++row;
        }
    }
    if (rs[0] == 0 || rs[2] + 1 >= jb.rows) return false;
    Src s[3];
    if (multi) { // all three descriptions are fetched before any is used
        FSTX_UNROLL
        for (int x = 0; x < 3; ++x) s[x] = src_uniform(more, jb.more0 + ks[x]);
    } else {
        s[0] = s[1] = s[2] = Src{jb.src, jb.pitch, jb.seg, 0, 0};
    }
    uint32_t pos[3], end[3];
    FSTX_UNROLL
    for (int x = 0; x < 3; ++x) {
        pos[x] = rs[x] * dst_pitch + s[x].col;
        end[x] = pos[x] + s[x].seg;
    }
    if (t_lo + kTile > end[2]) return false; // a fourth segment reaches into the tile
    // ---- per lane: which span, then the address (the vector units have time to spare)
    const uint32_t q = t_lo + kVec * lane; // position of the vector's byte 0
    const bool in_a = q < end[0], in_ab = q < end[1];
    const uint32_t end1 = in_a ? end[0] : in_ab ? end[1] : end[2];
    const uint32_t pos1 = in_a ? pos[0] : in_ab ? pos[1] : pos[2];
    const bool has2 = end1 < q + kVec; // the span ends inside the vector (never the third span's: the tile ends before it does)
    const uint32_t pos2 = in_a ? pos[1] : pos[2];
    if (kPitched && (q < pos1 || (has2 && pos2 != end1))) return false; // begins or continues in a gap: partly payload
    Vec16 g1, g2 = {{0, 0, 0, 0}};
    if (!kMulti) {
        // one source: the three spans are consecutive rows, position p of span x holds the byte at
        // base + x * step + p; two 64-bit values in scalar registers, one multiply-add per lane
        const char *base = jb.src + (uint64_t)rs[0] * jb.pitch - pos[0];
        const uint64_t step = jb.pitch - dst_pitch;
        const uint32_t x = (in_a ? 0u : 1u) + (in_ab ? 0u : 1u); // arithmetic, not a select: selects of scalar pairs become branches
        const char *base1 = base + x * step;
        g1 = mem.load16_stream(base1 + q);
        if (has2) g2 = mem.load16(base1 + step + q); // the next row begins end1 - q bytes into the vector
    } else {
        // several sources: the scalar unit already has the table to read, the address is put together per lane
        const uint32_t row1 = in_a ? rs[0] : in_ab ? rs[1] : rs[2];
        const char *src1 = in_a ? s[0].src : in_ab ? s[1].src : s[2].src;
        const uint64_t pitch1 = in_a ? s[0].pitch : in_ab ? s[1].pitch : s[2].pitch;
        g1 = mem.load16_stream(src1 + (uint64_t)row1 * pitch1 + (q - pos1));
        if (has2) { // the following span begins end1 - q bytes into the vector: the load starts that far before its first byte
            const uint32_t row2 = in_a ? rs[1] : rs[2];
            const char *src2 = in_a ? s[1].src : s[2].src;
            const uint64_t pitch2 = in_a ? s[1].pitch : s[2].pitch;
            g2 = mem.load16(src2 + (uint64_t)row2 * pitch2 - (pos2 - q));
        }
    }
    const uint32_t from2 = has2 ? end1 - q : kVec;
    mem.store16(jb.dst + q, blend(g1, g2, from2, kVec - from2));
    return true;
}

// One lane's work: vector `lane` of tile `tile` of job `jb`.
//
// A vector holds at most two parts (every segment is at least as long as a vector): the rest
// of the segment in which its first payload byte lies and, when that ends inside the vector,
// the beginning of the segment that follows -- in the same row, or in the next row behind the
// gap of a pitched destination.  The addresses of both parts are worked out first, then both
// loads are issued, and only then is either result looked at: a wavefront that contains a seam
// waits for memory once, like any other.  A load may reach up to 15 bytes beyond its segment on
// either side, into the neighbouring bytes of the source block (which the caller guarantees to
// be readable from the first segment's first byte to the last segment's last byte); at the two
// ends of the block it is pulled back inside and its result moved into place.
//
// kMulti: some job of the launch has more than one source; kPitched: some job's destination rows
// are further apart than their payload.  A launch without either (rank blocks of single tensors
// into dense destinations, the common case) runs the lean variant.
template <bool kMulti, bool kPitched, class Mem>
FSTX_HD void gather_lane(const Job &jb, const Src *more, uint32_t tile, uint32_t lane, Mem &mem) {
    if (gather_lane_inner<kMulti, kPitched>(jb, more, tile, lane, mem)) return;
    const uint32_t head = (uint32_t)((uintptr_t)jb.dst & (kVec - 1));
    const uint32_t dst_pitch = kPitched ? jb.dst_pitch : jb.row_bytes;
    // ---- once per wavefront (joins only): the segment at the start of the tile and the one after it
    Near near = {{0, 0, nullptr, nullptr, nullptr}, {0, 0, nullptr, nullptr, nullptr}, 0, 0};
    const bool by_rows = kPitched && (jb.flags & kByRows);
    if (kMulti && jb.nsrc > 1 && !by_rows) {
        const uint32_t t_lo = tile == 0 ? 0u : tile * kTile - head;
        near.row_a = t_lo / dst_pitch;
        uint32_t c0 = t_lo - near.row_a * dst_pitch;
        if (kPitched && c0 >= jb.row_bytes) { // the tile begins in a gap: the next row's first segment
            c0 = 0;
            ++near.row_a;
        }
        const uint32_t k = source_of(jb, more, c0);
        const uint32_t k2 = k + 1 < jb.nsrc ? k + 1 : 0u;
        near.row_b = k2 ? near.row_a : near.row_a + 1;
        // both descriptions are fetched before either is used
        const Src sa = src_uniform(more, jb.more0 + k);
        const Src sb = src_uniform(more, jb.more0 + k2);
        near.a = piece_from(sa.src, sa.pitch, sa.seg, sa.col, near.row_a, jb.rows);
        near.b = piece_from(sb.src, sb.pitch, sb.seg, sb.col, near.row_b, jb.rows);
    }
    // ---- per lane
    const uint32_t j = tile * kLanes + lane;
    if (j >= jb.nvec) return;
    char *out;
    uint32_t at, row, c;
    if (by_rows) {
        // vector v of row `row`: the 16 aligned bytes at align_down(the row's first byte, 16) + 16 v
        const uint32_t per_row = vectors_per_row(jb.row_bytes);
        row = j / per_row;
        const uint32_t v = j - row * per_row;
        char *row_dst = jb.dst + (uint64_t)row * dst_pitch;
        const uint32_t row_head = (uint32_t)((uintptr_t)row_dst & (kVec - 1));
        out = row_dst - row_head + kVec * v;
        at = v == 0 ? row_head : 0u;
        c = kVec * v - row_head + at;
        if (c >= jb.row_bytes) return; // beyond this row's last vector
    } else {
        out = jb.dst - head + (uint64_t)kVec * j;
        // pitched position p is destination byte dst + p: row p / dst_pitch, column p % dst_pitch
        at = j == 0 ? head : 0u;            // vector 0 begins `head` bytes before the job does
        const uint32_t q = kVec * j - head; // position of the vector's byte 0 (wraps for j == 0 when head > 0)
        row = (q + at) / dst_pitch;
        c = (q + at) - row * dst_pitch;
        if (kPitched && c >= jb.row_bytes) { // the vector begins in the gap behind a row's payload
            at += dst_pitch - c;
            c = 0;
            ++row;
        }
        if (at >= kVec || row >= jb.rows) return; // nothing of the job in this vector
    }
    // ---- part 1
    const Piece p1 = piece_of<kMulti>(jb, more, row, c, near);
    const uint32_t in1 = c - p1.col;
    const uint32_t at1 = at;
    const uint32_t take1 = p1.len - in1 < kVec - at1 ? p1.len - in1 : kVec - at1;
    const char *ideal1 = p1.bytes + in1 - at1; // where a load has to start to put the segment's byte in1 at byte at1
    const char *addr1 = ideal1 < p1.lo ? p1.lo : ideal1 + kVec > p1.hi ? p1.hi - kVec : ideal1;
    // ---- part 2
    uint32_t at2 = at1 + take1, c2 = c + take1, row2 = row;
    if (c2 == jb.row_bytes) { // the row's payload ends: over the gap (if any) into the next row
        if (kPitched) at2 += dst_pitch - jb.row_bytes;
        c2 = 0;
        ++row2;
    }
    const bool has2 = at2 < kVec && row2 < jb.rows;
    Vec16 g2 = {{0, 0, 0, 0}};
    const char *ideal2 = nullptr, *addr2 = nullptr;
    if (has2) {
        const Piece p2 = piece_of<kMulti>(jb, more, row2, c2, near); // c2 is a segment's first column
        ideal2 = p2.bytes - at2;
        addr2 = ideal2 < p2.lo ? p2.lo : ideal2; // (the vector ends inside the segment: it is at least a vector long)
    }
    // ---- both loads, then the arithmetic
    Vec16 g1 = mem.load16_stream(addr1);
    if (has2) g2 = mem.load16(addr2);
    const uint32_t from2 = has2 ? at2 : kVec; // bytes [from2, 16) come from part 2
    const bool plain = at1 == 0 && at1 + take1 >= from2 && addr1 == ideal1 && (!has2 || addr2 == ideal2);
    if (plain) {
        // nearly every vector, seams between segments included: straight-line code for the whole wavefront
        mem.store16(out, blend(g1, g2, from2, kVec - from2));
        return;
    }
    // the rest: the two ends of a source block (the load was pulled back inside it) and vectors
    // that are only partly the job's (its two ends, the gaps of a pitched destination)
    if (addr1 != ideal1) g1 = shifted(g1, (int32_t)(addr1 - ideal1));
    uint32_t mask = ((1u << take1) - 1u) << at1; // bit i: byte i of the vector is payload
    Vec16 acc = g1;
    if (has2) {
        if (addr2 != ideal2) g2 = shifted(g2, (int32_t)(addr2 - ideal2));
        acc = blend(acc, g2, at2, kVec - at2);
        mask |= 0xffffu & (0xffffu << at2);
    }
    if (mask == 0xffffu) {
        mem.store16(out, acc);
    } else {
        FSTX_UNROLL
        for (uint32_t i = 0; i < kVec; ++i)
            if (mask >> i & 1u) mem.store8(out + i, (unsigned char)(acc.w[i >> 2] >> (8 * (i & 3))));
    }
}

// ---- host side: the shapes the kernel takes, and how a job is cut to fit 32-bit positions

// Positions (bytes counted from the job's first, rows dst_pitch apart) are 32-bit in the kernel;
// a job may span this many at most, which leaves room for the tile that holds the last one.
constexpr uint64_t kMaxSpan = 0xffffffffull - 2 * kTile;

inline bool shape_ok(uint64_t dst_pitch, uint64_t row_bytes, uint64_t min_seg) {
    return min_seg >= kMinSeg && row_bytes <= dst_pitch && dst_pitch <= kMaxSpan;
}

// rows one job may cover (>= 1 when shape_ok)
inline uint64_t rows_per_job(uint64_t dst_pitch, uint64_t row_bytes) {
    return (kMaxSpan - row_bytes) / dst_pitch + 1;
}

// One source: `one` is it and more0 is unused.  Several: they sit at table[more0 .. more0 + nsrc)
// of the launch and `one` is ignored.
inline Job make_job(char *dst, uint64_t dst_pitch, uint64_t row_bytes, uint64_t rows, const Src &one, uint32_t more0,
                    uint32_t nsrc, uint64_t equal_seg, uint64_t min_seg) {
    const uint64_t head = (uint64_t)(uintptr_t)dst & (kVec - 1);
    const uint64_t span = (rows - 1) * dst_pitch + row_bytes;
    // one source into a pitched destination is always counted row by row from each row's own first
    // byte (no vector then holds a gap); several sources only when the gaps are a large part of the rows
    const bool single = nsrc == 1, loose = single && dst_pitch != row_bytes, by_rows = loose || counts_by_rows(dst_pitch, row_bytes);
    const uint32_t per_row = loose ? loose_vectors_per_row((uint32_t)row_bytes) : vectors_per_row((uint32_t)row_bytes);
    const uint64_t nvec = by_rows ? rows * per_row : (head + span + kVec - 1) / kVec;
    return Job{dst, (uint32_t)dst_pitch, (uint32_t)row_bytes, (uint32_t)rows, (uint16_t)more0, (uint16_t)nsrc,
               (uint32_t)nvec, (uint32_t)(single ? 0 : equal_seg), single ? one.src : nullptr,
               single ? one.pitch : magic_of(equal_seg), single ? one.seg : 0u,
               (by_rows ? kByRows : 0u) | (loose ? kLooseRows : 0u) | (min_seg < kShortSeg ? kShort : 0u),
               magic_of(by_rows ? per_row : dst_pitch)};
}

inline uint64_t tiles_of(const Job &jb) { return ((uint64_t)jb.nvec + kLanes - 1) / kLanes; }

} // namespace fstx_gather

#endif
