// Tile instance: 64 pixels x 64 features per workgroup, 16 pixels per wave.
#define TILE_BM 64
#define TILE_BN 64
#define TILE_WP 16
#define TILE_FN launch_mfma_tile_4
#include "conv_mfma_tile.inc"
