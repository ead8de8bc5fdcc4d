// The weight-streaming products reading the weight as it is stored, rows of K.
#include "gemm_skinny_impl.h"

void gs_skinny_plain_rows(const SkinnyCall& c) { skinny_plain<0>(c); }
void gs_skinny_residual_rows(const SkinnyCall& c) { skinny_residual<0>(c); }
void gs_skinny_conv_rows(const SkinnyCall& c) { skinny_conv<0>(c); }
void gs_skinny_parts_rows(const SkinnyCall& c, int parts) { skinny_parts<0>(c, parts); }
