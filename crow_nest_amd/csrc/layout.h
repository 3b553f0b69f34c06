// The tiled NVFP4 layout the gfx950 kernels read ("matrix-core tiles"), shared by host and device code.
//
// A container tensor [rows][cols] (cols % 64 == 0; 36-byte blocks of 4 UE4M3 scale bytes + 32
// code bytes, reference layout: engine/src/cpu_nvfp4.rs:8-18) is cut into tiles of
// 64 rows x 256 columns.  A tile is 9216 bytes and is read by ONE 64-lane wavefront with nine
// fully coalesced 16-byte-per-lane loads (each load instruction covers 1024 contiguous bytes).
// Inside a tile the bytes are placed so that what a lane loads IS its operand of the
// 16x16x32 bf16 matrix instruction (weight rows on the N side, 32 columns on the K side), with no
// exchange between lanes.  Lane l = 16 g + n  (g = 0..3, n = 0..15):
//
//   bytes 1024 (s + 1) + 16 l + 4 d .. + 3,   s = 0..7 (column segment), d = 0..3 (row group)
//       codes: the four code bytes (eight values, container order: byte j = value 2j in the low
//       nibble, 2j + 1 in the high one) of tile row 16 d + n, tile columns 32 s + 8 g .. + 7.
//       Dword d of load s is the B operand of the "unit" (row group d, segment s): lane (n, g)
//       holds column n of B for K indices 8 g .. 8 g + 7.
//   bytes 16 l + 8 jp + s,   jp = 0..1, s = 0..7
//       scales: the canonical scale byte of tile row 16 (2 jp + (g & 1)) + n, 16-column sub-block
//       2 s + (g >> 1) of the tile.  That is the scale a lane needs for the results it holds
//       after the GEMV's pair of matrix instructions on units (2 jp, s) and (2 jp + 1, s): lane
//       groups g = 0, 2 receive row group 2 jp (columns 0..15 and 16..31 of the segment), lane groups
//       g = 1, 3 row group 2 jp + 1.
//
// Tiles are stored row-tile major, then column panel: tile (rt, p) starts at
// (rt * panels + p) * 9216 with panels = ceil(cols / 256).  Rows beyond `rows` and columns beyond
// `cols` are zero (scale byte 0, code 0).  For rows % 64 == 0 and cols % 256 == 0 the tiled tensor
// has exactly the container's size (4.5 bits per weight).
//
// Scale bytes are canonicalised at repack time so that the hardware E4M3 decode reads the value
// the reference's CPU path computes with (engine/src/cpu_nvfp4.rs:88-105):
//   0x7F -> 0x7E   (the 0x7F -> 448 rule)
//   0x80..0xFE -> byte & 0x7F   (bit 7 is ignored by the reference decode, cnq.rs:1287-1295)
//   0xFF is refused (it reads 480 in the reference, which E4M3 cannot hold; no encoder emits it)
#pragma once
#include <stddef.h>
#include <stdint.h>

#define CROW_TILE_ROWS 64
#define CROW_PANEL_COLS 256
#define CROW_STEP_COLS 32
#define CROW_STEPS 8
#define CROW_TILE_SCALE_BYTES 1024
#define CROW_TILE_BYTES 9216
#define CROW_BLOCK_BYTES 36
#define CROW_BLOCK_VALUES 64

#ifdef __HIPCC__
#define CROW_HD __host__ __device__
#else
#define CROW_HD
#endif

// byte offset inside a tile of the code dword that holds tile row `row`, tile columns 8 wp .. 8 wp + 7 (wp = 0..31)
CROW_HD static inline unsigned crow_tile_code_offset(unsigned row, unsigned wp) {
    return 1024u * ((wp >> 2) + 1u) + 16u * (16u * (wp & 3u) + (row & 15u)) + 4u * (row >> 4);
}
// byte offset inside a tile of the scale byte of tile row `row`, sub-block sb (= tile column / 16, 0..15)
CROW_HD static inline unsigned crow_tile_scale_offset(unsigned row, unsigned sb) {
    const unsigned j = row >> 4, g = 2u * (sb & 1u) + (j & 1u);
    return 16u * (16u * g + (row & 15u)) + 8u * (j >> 1) + (sb >> 1);
}

static inline size_t crow_row_tiles(size_t rows) { return (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS; }
static inline size_t crow_panels(size_t cols) { return (cols + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS; }
static inline size_t crow_tiled_bytes(size_t rows, size_t cols) { return crow_row_tiles(rows) * crow_panels(cols) * CROW_TILE_BYTES; }
static inline size_t crow_container_bytes(size_t rows, size_t cols) { return rows * (cols / CROW_BLOCK_VALUES) * CROW_BLOCK_BYTES; }
