// Tile instance: 128 pixels x 64 features per workgroup, 32 pixels per wave.
#define TILE_BM 128
#define TILE_BN 64
#define TILE_WP 32
#define TILE_FN launch_mfma_tile_3
#include "conv_mfma_tile.inc"
