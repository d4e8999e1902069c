// Tile instance: 256 pixels x 64 features per workgroup, 64 pixels per wave.
#define TILE_BM 256
#define TILE_BN 64
#define TILE_WP 64
#define TILE_FN launch_mfma_tile_1
#include "conv_mfma_tile.inc"
