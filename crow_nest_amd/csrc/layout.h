// The tiled NVFP4 layout the gfx950 kernels read ("lane-row tiles"), shared by host and device code.
//
// A container tensor [rows][cols] (cols % 64 == 0; 36-byte blocks of 4 UE4M3 scale bytes + 32
// code bytes, reference layout: engine/src/cpu_nvfp4.rs:8-18) is cut into tiles of
// 64 rows x 256 columns.  A tile is 9216 bytes and is read by ONE 64-lane wavefront with nine
// fully coalesced 16-byte-per-lane loads (each load instruction covers 1024 contiguous bytes):
//
//   bytes    0 .. 1023   scales: lane l (= row l of the tile) owns bytes 16 l .. 16 l + 15, the
//                        scale bytes of its 16 sub-blocks (16 values each), canonicalised
//   bytes 1024 (s + 1) + 16 l .. + 15,  s = 0..7
//                        codes: the 16 code bytes of row l for columns 32 s .. 32 s + 31 of the
//                        tile, in container order (byte j: value 2j low nibble, 2j + 1 high)
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

static inline size_t crow_row_tiles(size_t rows) { return (rows + CROW_TILE_ROWS - 1) / CROW_TILE_ROWS; }
static inline size_t crow_panels(size_t cols) { return (cols + CROW_PANEL_COLS - 1) / CROW_PANEL_COLS; }
static inline size_t crow_tiled_bytes(size_t rows, size_t cols) { return crow_row_tiles(rows) * crow_panels(cols) * CROW_TILE_BYTES; }
static inline size_t crow_container_bytes(size_t rows, size_t cols) { return rows * (cols / CROW_BLOCK_VALUES) * CROW_BLOCK_BYTES; }
