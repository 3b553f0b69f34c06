// The NVFP4 layout the gfx950 kernels read ("row strips of matrix-core groups"), shared by host and device code.
//
// A container tensor [rows][cols] (cols % 64 == 0; 36-byte blocks of 4 UE4M3 scale bytes + 32 code bytes, reference
// layout: engine/src/cpu_nvfp4.rs:8-18) is cut into STRIPS of 16 rows, and every strip into GROUPS of 256 columns.  A
// group is 2304 bytes - exactly the container bytes of its 16 x 256 values - and a strip's groups are contiguous in
// column order, strips in row order: group (strip, gi) starts at (strip * groups + gi) * 2304 with
// groups = ceil(cols / 256).  A wavefront that owns n consecutive groups of a strip reads n * 2304 contiguous bytes with
// fully coalesced loads, and whatever a lane loads IS its operand of the 16x16x32 bf16 matrix instruction (the 16 weight
// rows on the N side, 32 columns on the K side), with no exchange between lanes.  Because a strip is only 16 rows tall, all
// columns of a strip fit the waves of ONE workgroup for any K up to 16384: the GEMVs then reduce in LDS only.
//
// Inside a group, lane l = 16 g + n (g = 0..3, n = 0..15); a PAIR is 64 columns = two 32-column segments:
//
//   bytes 256 + 1024 h + 16 l + 4 d .. + 3,   h = 0..1, d = 0..3
//       codes: the four code bytes (eight values, container order: byte j = value 2 j in the low nibble, 2 j + 1 in the
//       high one) of strip row n, group columns 64 (2 h + (d >> 1)) + 32 (d & 1) + 8 g .. + 7.  So the 16 bytes a lane loads
//       from half h are pairs 2 h and 2 h + 1, and dword d is the B operand of pair 2 h + (d >> 1), segment d & 1: lane (n, g)
//       holds column n of B for K indices 8 g .. 8 g + 7.
//   bytes 4 l + jj,   jj = 0..3 (pair)
//       scales: the canonical scale byte of strip row n, 16-column sub-block 4 jj + 2 (g & 1) + (g >> 1) of the group
//       (columns 64 jj + 32 (g & 1) + 16 (g >> 1) .. + 15).  That is the scale a lane needs for the result it holds after the
//       GEMV's two matrix instructions on pair jj (gemv.h): lane groups g = 0, 2 receive segment 0 of the pair (its columns
//       0..15 and 16..31), lane groups g = 1, 3 segment 1.
//
// Rows beyond `rows` and columns beyond `cols` are zero (scale byte 0, code 0).  For rows % 16 == 0 and cols % 256 == 0
// the tensor has exactly the container's size (4.5 bits per weight).
//
// Scale bytes are canonicalised at repack time so that the hardware E4M3 decode reads the value
// the reference's CPU path computes with (engine/src/cpu_nvfp4.rs:88-105):
//   0x7F -> 0x7E   (the 0x7F -> 448 rule)
//   0x80..0xFE -> byte & 0x7F   (bit 7 is ignored by the reference decode, cnq.rs:1287-1295)
//   0xFF is refused (it reads 480 in the reference, which E4M3 cannot hold; no encoder emits it)
#pragma once
#include <stddef.h>
#include <stdint.h>

#define CROW_STRIP_ROWS 16
#define CROW_GROUP_COLS 256
#define CROW_GROUP_PAIRS 4
#define CROW_PAIR_COLS 64
#define CROW_GROUP_SCALE_BYTES 256
#define CROW_GROUP_BYTES 2304
#define CROW_BLOCK_BYTES 36
#define CROW_BLOCK_VALUES 64

#ifdef __HIPCC__
#define CROW_HD __host__ __device__
#else
#define CROW_HD
#endif

// byte offset inside a group of the code dword that holds strip row `row` (0..15), group columns 8 wp .. 8 wp + 7 (wp = 0..31)
CROW_HD static inline unsigned crow_group_code_offset(unsigned row, unsigned wp) {
    const unsigned pair = wp >> 3, seg = (wp >> 2) & 1u, g = wp & 3u;
    return 256u + 1024u * (pair >> 1) + 16u * (16u * g + row) + 4u * (2u * (pair & 1u) + seg);
}
// byte offset inside a group of the scale byte of strip row `row` (0..15), sub-block sb (= group column / 16, 0..15)
CROW_HD static inline unsigned crow_group_scale_offset(unsigned row, unsigned sb) {
    const unsigned pair = sb >> 2, seg = (sb >> 1) & 1u, half = sb & 1u;
    return 4u * (16u * (2u * half + seg) + row) + pair;
}

static inline size_t crow_strips(size_t rows) { return (rows + CROW_STRIP_ROWS - 1) / CROW_STRIP_ROWS; }
static inline size_t crow_groups(size_t cols) { return (cols + CROW_GROUP_COLS - 1) / CROW_GROUP_COLS; }
static inline size_t crow_tiled_bytes(size_t rows, size_t cols) { return crow_strips(rows) * crow_groups(cols) * CROW_GROUP_BYTES; }
static inline size_t crow_container_bytes(size_t rows, size_t cols) { return rows * (cols / CROW_BLOCK_VALUES) * CROW_BLOCK_BYTES; }
