// Tile instance: 256 pixels x 128 features per workgroup, 128 pixels per wave.
#define TILE_BM 256
#define TILE_BN 128
#define TILE_WP 128
#define TILE_FN launch_mfma_tile_5
#include "conv_mfma_tile.inc"
