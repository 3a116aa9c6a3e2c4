// Geometry of the gather maps and their internal launchers (the exported entry points check their
// arguments and call these; the DeConv2d operators call them with a mirrored geometry).
#ifndef DEEP8_AMD_CONV_MAPS_H
#define DEEP8_AMD_CONV_MAPS_H

#include "common.h"

namespace d8 {

// Patch row (b, oy, ox) of an OH x OW grid, tap (fy, fx), reads image pixel
// (oy * sy + fy * dy - pt, ox * sx + fx * dx - pl) of a [B][IH][IW][C] image.  dy, dx, pt, pl may
// be negative (the DeConv2d maps are this map with dy = dx = -1 and negated pads).
struct MapGeom {
    int B, IH, IW, C, OH, OW, FH, FW, sy, sx, dy, dx, pt, pl;
    int pitch;  // elements from one row of col to the next; 0: FH * FW * C (dense).  im2col zeroes the padding.
};

// col[(b,oy,ox)][(fy,fx,c)] = image pixel or 0
int launch_im2col(int dtype, const void *im, void *col, const MapGeom &g, hipStream_t stream);
// im (+)= the transpose of that map applied to col; taps added in (fy, fx) ascending order
int launch_col2im(int dtype, const void *col, void *im, const MapGeom &g, bool accumulate, hipStream_t stream);

// dst[r][0 .. K) = src[r][0 .. K), dst[r][K .. pitch) = 0: a matrix copied into a row pitch that 16-byte loads can use
int launch_pad_rows(int dtype, const void *src, void *dst, long rows, int K, int pitch, hipStream_t stream);
// the way back: dst[r][0 .. K) = beta * dst[r][0 .. K) + src[r][0 .. K) of a matrix with row pitch `pitch`
int launch_unpad_add(int dtype, const void *src, void *dst, long rows, int K, int pitch, float beta, hipStream_t stream);

}  // namespace d8

#endif
