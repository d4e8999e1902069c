// Tile instance: 64 pixels x 128 features per workgroup, 32 pixels per wave.
#define TILE_BM 64
#define TILE_BN 128
#define TILE_WP 32
#define TILE_FN launch_mfma_tile_2
#include "conv_mfma_tile.inc"
