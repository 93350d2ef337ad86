// The 𝚒 runtime C ABI (include/i.h): component handles and combinators.
// Reference behaviour: core/src/lib.rs:61-121, 289-351.
#include "../../../include/i.h"

#include <cstdlib>
#include <cstring>
#include <string>

#include "error.h"
#include "handles.h"

namespace {

i_component* wrap(ic::Component c) { return new i_component{std::make_shared<const ic::Component>(std::move(c))}; }

i_component* combine(const i_component* left, const i_component* right, ic::Component::Kind kind) {
  if (!left) {
    icore::set_error("null left component");
    return nullptr;
  }
  if (!right) {
    icore::set_error("null right component");
    return nullptr;
  }
  ic::Component c;
  c.kind = kind;
  c.a = left->inner;  // component trees are immutable, so sharing is a clone
  c.b = right->inner;
  return wrap(std::move(c));
}

// Strict UTF-8 check, matching CStr::to_str in the reference's read_str.
bool valid_utf8(const char* s) {
  const unsigned char* p = reinterpret_cast<const unsigned char*>(s);
  while (*p) {
    int n = *p < 0x80 ? 0 : (*p >> 5) == 0x6 ? 1 : (*p >> 4) == 0xE ? 2 : (*p >> 3) == 0x1E ? 3 : -1;
    if (n < 0) return false;
    if (n == 1 && *p < 0xC2) return false;
    ++p;
    for (int i = 0; i < n; ++i, ++p)
      if ((*p & 0xC0) != 0x80) return false;
  }
  return true;
}

}  // namespace

extern "C" {

i_component* i_parse(const char* src) {
  if (!src || !valid_utf8(src)) {
    icore::set_error("null source");
    return nullptr;
  }
  try {
    ic::Component c;
    c.kind = ic::Component::Leaf;
    c.expr = ic::parse_expr(src);
    return wrap(std::move(c));
  } catch (const ic::CompileError& e) {
    icore::set_error(e.debug_string());
  } catch (const std::exception& e) {
    icore::set_error(e.what());
  }
  return nullptr;
}

i_component* i_identity(void) { return wrap(ic::Component{}); }

i_component* i_chain(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Chain); }
i_component* i_compose(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Compose); }
i_component* i_fanout(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Fanout); }
i_component* i_pair(const i_component* l, const i_component* r) { return combine(l, r, ic::Component::Pair); }

i_component* i_swap(const i_component* component) {
  if (!component) {
    icore::set_error("null component");
    return nullptr;
  }
  ic::Component c;
  c.kind = ic::Component::Swap;
  c.a = component->inner;
  return wrap(std::move(c));
}

void i_component_free(i_component* component) { delete component; }

void i_string_free(char* s) { std::free(s); }

const char* i_error(void) { return icore::last_error(); }

}  // extern "C"
