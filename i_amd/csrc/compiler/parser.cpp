// Recursive-descent parser for one 𝚒 expression  "semantic | splits | order".
// Grammar, token table and error texts follow compiler/src/front/parser.rs:48-296.
#include <cctype>

#include "ir.h"

namespace ic {
namespace {

struct Parser {
  const std::string& src;
  size_t pos = 0;
  explicit Parser(const std::string& s) : src(s) {}

  [[noreturn]] void fail(const std::string& message) const { throw CompileError("ParseError", message, pos); }
  int peek() const { return pos < src.size() ? (unsigned char)src[pos] : -1; }
  bool eof() const { return pos >= src.size(); }
  static bool lower(int c) { return c >= 'a' && c <= 'z'; }
  static bool digit(int c) { return c >= '0' && c <= '9'; }
  void skip_ws() {
    while (pos < src.size()) {
      const char c = src[pos];
      if (c == ' ' || c == '\t' || c == '\n' || c == '\r' || c == '\f') ++pos;  // u8::is_ascii_whitespace
      else break;
    }
  }
  bool consume_if(char c) {
    skip_ws();
    if (peek() == c) { ++pos; return true; }
    return false;
  }
  void expect(char c, const char* message) {
    skip_ws();
    if (peek() == c) ++pos;
    else fail(message);
  }

  bool parse_op(Op& op) {
    skip_ws();
    static const std::pair<const char*, Op> table[] = {
        {">>", Op::Gt}, {">=", Op::Ge}, {"<<", Op::Lt}, {"<=", Op::Le}, {"==", Op::Eq}, {"!=", Op::Ne},
        {"&&", Op::And}, {"||", Op::Or}, {"^^", Op::Xor}, {"!!", Op::Not}, {"+", Op::Add}, {"*", Op::Mul},
        {"-", Op::Sub}, {"/", Op::Div}, {">", Op::Max}, {"<", Op::Min}, {"^", Op::Pow}, {"$", Op::Log}};
    for (const auto& [token, value] : table) {
      const size_t n = std::char_traits<char>::length(token);
      if (src.compare(pos, n, token) == 0) {
        pos += n;
        op = value;
        return true;
      }
    }
    return false;
  }

  std::vector<char> parse_pattern() {
    skip_ws();
    if (peek() == '.') {
      ++pos;
      if (lower(peek()) || peek() == '.') fail("scalar pattern must be `.`");
      return {};
    }
    std::vector<char> axes;
    while (lower(peek())) axes.push_back(src[pos++]);
    if (axes.empty()) fail("expected pattern");
    return axes;
  }

  char parse_axis() {
    skip_ws();
    if (lower(peek())) return src[pos++];
    fail("expected axis");
  }

  size_t parse_usize() {
    skip_ws();
    const size_t start = pos;
    while (digit(peek())) ++pos;
    if (pos == start) fail("expected integer");
    size_t value = 0;
    for (size_t i = start; i < pos; ++i) {
      const size_t d = src[i] - '0';
      if (value > (SIZE_MAX - d) / 10) throw CompileError("ParseError", "invalid integer", start);
      value = value * 10 + d;
    }
    return value;
  }

  std::vector<std::pair<char, std::vector<size_t>>> parse_splits() {
    std::vector<std::pair<char, std::vector<size_t>>> splits;
    for (;;) {
      const char axis = parse_axis();
      expect(':', "expected `:` after split axis");
      std::vector<size_t> factors{parse_usize()};
      while (consume_if(':')) factors.push_back(parse_usize());
      for (const auto& s : splits)
        if (s.first == axis) fail(std::string("duplicate split entry for axis ") + axis);
      splits.emplace_back(axis, factors);
      if (!consume_if(',')) break;
    }
    return splits;
  }

  std::vector<PermAtom> parse_permutation() {
    std::vector<PermAtom> perm;
    bool seen_input[2] = {false, false};
    bool seen_bang = false;
    for (;;) {
      skip_ws();
      if (eof()) break;
      if (lower(peek())) {
        PermAtom a;
        a.kind = PermAtom::Axis;
        a.axis = parse_axis();
        while (consume_if('\'')) ++a.part;
        perm.push_back(a);
        continue;
      }
      if (digit(peek())) {
        skip_ws();
        size_t operand;
        if (peek() == '0') operand = 0;
        else if (peek() == '1') operand = 1;
        else fail("expected operand `0` or `1`");
        ++pos;
        if (seen_input[operand]) fail("duplicate compute directive for input " + std::to_string(operand));
        seen_input[operand] = true;
        PermAtom a;
        a.kind = PermAtom::Input;
        a.operand = operand;
        perm.push_back(a);
        continue;
      }
      if (consume_if('!')) {
        if (seen_bang) fail("duplicate output init directive");
        seen_bang = true;
        PermAtom a;
        a.kind = PermAtom::Bang;
        perm.push_back(a);
        continue;
      }
      fail("expected axis, `!`, or operand in permutation");
    }
    return perm;
  }

  Expr parse_inner() {
    Expr e;
    Op op;
    if (parse_op(op)) {
      e.op = op;
      e.inputs.push_back(parse_pattern());
    } else {
      auto first = parse_pattern();
      skip_ws();
      if (peek() == '~') {
        e.op = Op::Add;
        e.inputs.push_back(first);
      } else {
        if (!parse_op(op)) fail("expected operator after input pattern");
        e.op = op;
        auto second = parse_pattern();
        e.inputs.push_back(first);
        e.inputs.push_back(second);
      }
    }
    skip_ws();
    expect('~', "expected `~` between inputs and output");
    e.output = parse_pattern();
    if (consume_if('|')) {
      skip_ws();
      if (peek() != '|') e.splits = parse_splits();
      expect('|', "expected second `|` in schedule");
      e.permutation = parse_permutation();
    }
    return e;
  }

  Expr parse_top() {
    skip_ws();
    if (eof()) fail("expected i-expression");
    Expr e = parse_inner();
    skip_ws();
    if (!eof()) fail("unexpected trailing input");
    return e;
  }
};

}  // namespace

Expr parse_expr(const std::string& src) { return Parser(src).parse_top(); }

}  // namespace ic
