// Tile bookkeeping shared by the tiled forward and backward kernels.
//
// The feature map of every image is cut into TH x TW pixel tiles.  A small
// pre-pass turns the ROI list into (a) one box record per ROI and (b) for
// every tile the ordered list of ROIs that have at least one sample corner in
// it.  The backward kernel is a "tile owner": one workgroup per (tile, channel
// block) keeps that piece of the map in LDS and walks the tile's work lists.
#pragma once
#include "roialign_geometry.h"

namespace roialign {

struct TileGrid {
  int th, tw;        // tile size in pixels
  int ty, tx;        // tiles per image along y and x
  int per_image;     // ty * tx
  long long total;   // per_image * num_images
};

// The tiles a list item (a ROI, or one window of its merged weights) touches: image
// (-1: none), first | last << 16 tile row, first | last << 16 tile column; and
// the ROI it belongs to.
struct alignas(16) TileBox { int batch; int ty; int tx; int roi; };

}  // namespace roialign
