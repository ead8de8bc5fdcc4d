// The weight-streaming products reading the tile-major copy of the weight.
#include "gemm_skinny_impl.h"

void gs_skinny_plain_tiles(const SkinnyCall& c) { skinny_plain<1>(c); }
void gs_skinny_residual_tiles(const SkinnyCall& c) { skinny_residual<1>(c); }
void gs_skinny_residual_half_tiles(const SkinnyCall& c) { skinny_residual<2>(c); }
void gs_skinny_conv_tiles(const SkinnyCall& c) { skinny_conv<1>(c); }
void gs_skinny_conv_half_tiles(const SkinnyCall& c) { skinny_conv<2>(c); }
void gs_skinny_parts_tiles(const SkinnyCall& c, int parts) { skinny_parts<1>(c, parts); }
