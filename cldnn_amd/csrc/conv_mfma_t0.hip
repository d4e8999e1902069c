// Tile instance: 128 pixels x 128 features per workgroup, 64 pixels per wave.
#define TILE_BM 128
#define TILE_BN 128
#define TILE_WP 64
#define TILE_FN launch_mfma_tile_0
#include "conv_mfma_tile.inc"
