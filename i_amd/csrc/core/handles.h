// The opaque handle types behind the C ABI.
#pragma once
#include "../compiler/ir.h"

struct i_component {
  ic::ComponentPtr inner;
};
