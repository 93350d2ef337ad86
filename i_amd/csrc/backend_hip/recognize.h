// Maps fused kernels of a lowered component onto the hand-written gfx950 kernels.
//
// After fusion every kernel is a tree of stages rooted at the stage that owns
// the kernel's loops; producers staged under a consumer are interior nodes and
// everything else is an operand buffer.  The tree, with the index symbols of
// producer and consumer unified along each edge, states WHAT the kernel
// computes independently of its loop order and splits.  Kernels whose tree is
// one of the known forms run on a hand-written kernel; all others go through
// the generic HIP emitter.
#pragma once
#include <string>
#include <vector>

#include "../compiler/ir.h"

namespace ihipc {

struct Operand {
  ic::BufferRef buffer;        // exec-plan buffer
  std::vector<int> dims;       // index symbols, outermost first
};

struct Recognized {
  enum Kind { None, Attention, GemmNT, GemmNN, RowSoftmax, RowMaxShift, RowNormalize, RowExp } kind = None;
  // Attention: q [B.., I, D], k [B.., J, D], v [B.., J, E] -> out [B.., I, E]; optional scalar scale
  // GemmNT:    a [B.., I, K], b [B.., J, K] -> out [B.., I, J]
  // GemmNN:    a [B.., I, K], b [B.., K, J] -> out [B.., I, J]
  // RowSoftmax, RowMaxShift (x - max_J x), RowNormalize (x / sum_J x), RowExp (exp x, elementwise):
  //            x [R.., J] -> out [R.., J]
  Operand a, b, c;             // q,k,v | a,b,- | x,-,-
  bool has_scale = false;
  Operand scale;               // rank-0 operand
  ic::BufferRef out;
  size_t batch_rank = 0;       // number of leading shared dims
  // Tile sizes the schedule asks for (product of the split factors of the index in the kernel's root
  // stage, 0 when the index is not split): Attention: query rows I / keys J; GemmNT, GemmNN: rows I / columns J.
  size_t tile_i = 0, tile_j = 0;
  std::string describe() const;
};

// One entry per kernel of `low.plan.kernels`.
std::vector<Recognized> recognize_kernels(const ic::Lowered& low);

}  // namespace ihipc
