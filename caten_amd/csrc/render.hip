// Hip-Renderer behind the C ABI: a Schedule-Item's blueprint, printed as an s-expression, becomes a PROGRAM --
// HIP source with gfx950-aware work distribution for the item, plus, where the item is one of the shapes a
// hand-written kernel covers, a route to that kernel.  Caten's renderer protocol (`%render-kernel` /
// `%compile-kernel`, source/codegen/renderer.lisp:30-34) is implemented by Lisp classes; the Lisp side of this
// backend (and the Python mirror the tests drive) only prints the blueprint and calls the entry points below, so
// both get the same kernels.
//
// Interchange text (case-insensitive; what a Lisp `format` of the Render-IR nodes of renderer.lisp:36-92 and
// aasm/attrs.lisp:298-318 gives):
//   (item NAME node...)
//   node := (define-global ID DTYPE POINTER-P input|output|shape NRANK)
//         | (for IDX UPFROM BELOW BY [local|global]) | (endfor IDX) | (if COND) | (endif)
//         | (expr (WRITE...) RHS :dtype DTYPE [:declare t] [:reduction t] [:grid (RANK GLOBAL-SIZE LOCAL-SIZE)])
//   WRITE, expr := number | inf | -inf | nan | t | nil | SYMBOL | (aref ID [INDEX]) | (const VALUE DTYPE)
//         | (cast DTYPE expr) | (space block|thread RANK) | (OP expr...)     OP = the aasm instruction set
// :grid marks the statement that binds an index to (space block RANK) * LOCAL-SIZE + (space thread RANK) after the
// auto-scheduler's GLOBAL directive (its ExprGrid); such an item is launched with exactly those sizes.
// BELOW is the loop condition, e.g. (< _gid0 n) (source/byoc/clang.lisp:58-73); an aref's INDEX is the flat element
// index sum_d stride_d * (from_d + by_d * gid_d) the reference renders (clang.lisp:82-97).
//
// Work distribution of rendered kernels (the reference leaves every loop serial at OPTIMIZE=1, so its Metal
// kernels run in one thread, source/byoc/metal.lisp:341-345): the outermost perfectly nested loops whose index
// appears in every global write below them are data-parallel and become one flat thread id, innermost fastest, in
// 256-thread workgroups; row reductions (a parallel prefix whose body is scalar statements and loops over one
// more axis, some of them reductions into scalars that start at the operation's identity) get one WAVEFRONT per
// row: the 64 lanes stride the axis together, partials meet in a __shfl_xor butterfly, lane 0 stores per-row
// scalars; a row of static length becomes counted, unrolled loops so that the row is read once.
//
// Routes (checked again at every launch against the actual shapes; anything that does not fit runs the rendered
// kernel): the matmul nest ADD(reduction) o MUL of source/test-suite/test-scheduler.lisp:126-135 with an
// optional bias / ReLU epilogue -> the MFMA GEMM (B row-major, or read through a transposed view as Linear does,
// source/nn/linear.lisp:3-17; fewer than eight rows of a Linear -> the single-row kernels); the one-hot masked sum
// of Embedding (source/nn/embedding.lisp:13-25) -> a row gather; ArgMaxNode's two reductions
// (source/api/high-level-ops.lisp:314-325) -> the argmax kernel; softmax rows (source/nn/activations.lisp:107-119)
// -> the row kernel.
#include <math.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <functional>
#include <map>
#include <string>
#include <vector>

#include "common.h"

namespace cthip {

// ------------------------------------------------------------------ s-expressions
struct Sx {
  enum Kind { LIST, SYM, INT, FLT, STR } kind = LIST;
  std::string s;       // SYM (lower case) / STR
  long long i = 0;     // INT
  double f = 0.0;      // FLT
  std::vector<Sx> v;   // LIST
  bool is_sym(const char *name) const { return kind == SYM && s == name; }
  bool is_list() const { return kind == LIST; }
  bool is_num() const { return kind == INT || kind == FLT; }
  const Sx &head() const { return v[0]; }
  bool call(const char *op) const { return kind == LIST && !v.empty() && v[0].is_sym(op); }
  size_t n() const { return v.size(); }
};
static Sx sx_sym(const std::string &s) { Sx x; x.kind = Sx::SYM; x.s = s; return x; }
static Sx sx_int(long long i) { Sx x; x.kind = Sx::INT; x.i = i; return x; }
static Sx sx_list(std::vector<Sx> v) { Sx x; x.kind = Sx::LIST; x.v = std::move(v); return x; }

struct Parser {
  const char *p;
  std::string err;
  void skip() {
    for (;;) {
      while (*p == ' ' || *p == '\n' || *p == '\t' || *p == '\r') p++;
      if (*p == ';') while (*p && *p != '\n') p++;
      else break;
    }
  }
  // Every later pass (rendering, probing, matching) recurses over the tree this builds, so the depth is bounded here:
  // no item of a real graph nests anywhere near this deep, and text that does must not run the host out of stack.
  static constexpr int kMaxDepth = 256;
  int depth = 0;
  bool parse(Sx &out) {
    skip();
    if (!*p) return err = "unexpected end of text", false;
    if (*p == '(') {
      if (depth >= kMaxDepth) return err = "lists nested deeper than 256", false;
      p++;
      depth++;
      out = Sx();
      for (;;) {
        skip();
        if (!*p) return err = "unbalanced '('", false;
        if (*p == ')') { p++; depth--; return true; }
        Sx e;
        if (!parse(e)) return false;
        out.v.push_back(std::move(e));
      }
    }
    if (*p == ')') return err = "unexpected ')'", false;
    if (*p == '"') {
      p++;
      out = Sx();
      out.kind = Sx::STR;
      while (*p && *p != '"') {
        if (*p == '\\' && p[1]) p++;
        out.s.push_back(*p++);
      }
      if (*p != '"') return err = "unterminated string", false;
      p++;
      return true;
    }
    std::string tok;
    while (*p && *p != ' ' && *p != '\n' && *p != '\t' && *p != '\r' && *p != '(' && *p != ')') tok.push_back(*p++);
    if (!tok.empty() && tok[0] == ':') tok = tok.substr(1);  // keywords and symbols are the same thing here
    std::string low;
    for (char c : tok) low.push_back((char)tolower((unsigned char)c));
    // numbers: integers, floats (Lisp prints 1.0d0 / 1.0f0 / 1.0e-5 exponent markers)
    std::string num = low;
    for (char &c : num) if (c == 'd' || c == 'f') c = 'e';
    char *end = nullptr;
    out = Sx();
    if (low == "inf" || low == "+inf") { out.kind = Sx::FLT; out.f = INFINITY; return true; }
    if (low == "-inf") { out.kind = Sx::FLT; out.f = -INFINITY; return true; }
    if (low == "nan") { out.kind = Sx::FLT; out.f = NAN; return true; }
    const bool numeric_start = !num.empty() && (isdigit((unsigned char)num[0]) || ((num[0] == '-' || num[0] == '+' || num[0] == '.') && num.size() > 1 && (isdigit((unsigned char)num[1]) || num[1] == '.')));
    if (numeric_start) {
      long long iv = strtoll(num.c_str(), &end, 10);
      if (end && !*end) { out.kind = Sx::INT; out.i = iv; return true; }
      double fv = strtod(num.c_str(), &end);
      if (end && !*end) { out.kind = Sx::FLT; out.f = fv; return true; }
    }
    out.kind = Sx::SYM;
    out.s = low;
    return true;
  }
};

// ------------------------------------------------------------------ blueprint
struct Global {
  std::string id, dtype, type;  // type: input / output / shape
  bool pointer = false;
  int nrank = 0;
};
struct BpNode {
  enum T { FOR, ENDFOR, IF, ENDIF, EXPR } t = EXPR;
  std::string idx;              // FOR / ENDFOR
  Sx upfrom, below, by;         // FOR
  bool global_scope = false;    // FOR
  Sx cond;                      // IF
  std::vector<Sx> writes;       // EXPR
  Sx rhs;
  bool declare = false, reduction = false;
  std::string dtype = "float32";
  // an index bound to blockIdx / threadIdx by the auto-scheduler's GLOBAL directive carries the launch size of
  // its axis (ExprGrid: source/codegen/auto-scheduler/directive.lisp:94-117, gathered by blueprint-gather-grids,
  // source/codegen/blueprint.lisp:726-737): rank 0..2, workgroups along it, threads per workgroup along it
  int grid_rank = -1;
  Sx grid_global, grid_local;
};
struct Item {
  std::string name;
  std::vector<Global> globals;
  std::vector<BpNode> body;
};

static const std::map<std::string, std::string> &cdtypes() {  // ->cdtype (source/codegen/helpers.lisp:101-113)
  static const std::map<std::string, std::string> m = {
      {"bool", "bool"}, {"float64", "double"}, {"float32", "float"}, {"float16", "_Float16"},
      {"uint64", "unsigned long long"}, {"int64", "long long"}, {"uint32", "unsigned int"}, {"int32", "int"},
      {"uint16", "unsigned short"}, {"int16", "short"}, {"uint8", "unsigned char"}, {"int8", "signed char"}};
  return m;
}
static size_t dtype_bytes(const std::string &d) {
  if (d == "float64" || d == "uint64" || d == "int64") return 8;
  if (d == "float32" || d == "uint32" || d == "int32") return 4;
  if (d == "float16" || d == "uint16" || d == "int16") return 2;
  return 1;
}

static bool truthy(const Sx &x) { return !(x.is_sym("nil") || (x.kind == Sx::LIST && x.v.empty())); }

static bool build_item(const Sx &top, Item &it, std::string &err) {
  if (!top.call("item") || top.n() < 2) return err = "expected (item NAME node...)", false;
  it.name = top.v[1].s;
  for (char &c : it.name) c = (char)tolower((unsigned char)c);
  if (it.name.empty()) return err = "the item has no name", false;
  int depth = 0, ifs = 0;
  for (size_t k = 2; k < top.n(); k++) {
    const Sx &n = top.v[k];
    if (!n.is_list() || n.v.empty() || n.v[0].kind != Sx::SYM) return err = "a blueprint node must be a list headed by its type", false;
    const std::string &ty = n.v[0].s;
    if (ty == "define-global") {
      if (n.n() != 6) return err = "(define-global ID DTYPE POINTER-P TYPE NRANK)", false;
      Global g;
      g.id = n.v[1].s;
      g.dtype = n.v[2].s;
      g.pointer = truthy(n.v[3]);
      g.type = n.v[4].s;
      g.nrank = (int)n.v[5].i;
      if (!cdtypes().count(g.dtype)) return err = "define-global: unknown dtype " + g.dtype, false;
      if (g.type != "input" && g.type != "output" && g.type != "shape") return err = "define-global: type is input, output or shape", false;
      it.globals.push_back(g);
    } else if (ty == "for") {
      if (n.n() < 5) return err = "(for IDX UPFROM BELOW BY [SCOPE])", false;
      BpNode b;
      b.t = BpNode::FOR;
      b.idx = n.v[1].s;
      b.upfrom = n.v[2];
      b.below = n.v[3];
      b.by = n.v[4];
      // a loop that does not advance would never leave its kernel
      if ((b.by.kind == Sx::INT && b.by.i < 1) || (b.by.kind == Sx::FLT && !(b.by.f >= 1.0)))
        return err = "for: the step must be at least 1", false;
      if (n.v[1].kind != Sx::SYM || n.v[1].s.empty()) return err = "for: the index must be a symbol", false;
      b.global_scope = n.n() > 5 && n.v[5].is_sym("global");
      it.body.push_back(b);
      depth++;
    } else if (ty == "endfor") {
      BpNode b;
      b.t = BpNode::ENDFOR;
      b.idx = n.n() > 1 ? n.v[1].s : "";
      it.body.push_back(b);
      if (--depth < 0) return err = "endfor without for", false;
    } else if (ty == "if") {
      if (n.n() != 2) return err = "(if COND)", false;
      BpNode b;
      b.t = BpNode::IF;
      b.cond = n.v[1];
      it.body.push_back(b);
      ifs++;
    } else if (ty == "endif") {
      BpNode b;
      b.t = BpNode::ENDIF;
      it.body.push_back(b);
      if (--ifs < 0) return err = "endif without if", false;
    } else if (ty == "expr") {
      if (n.n() < 3 || !n.v[1].is_list()) return err = "(expr (WRITE...) RHS :dtype DTYPE [:declare t] [:reduction t])", false;
      BpNode b;
      b.t = BpNode::EXPR;
      b.writes = n.v[1].v;
      b.rhs = n.v[2];
      for (size_t q = 3; q + 1 < n.n(); q += 2) {
        if (n.v[q].is_sym("dtype")) b.dtype = n.v[q + 1].s;
        else if (n.v[q].is_sym("declare") || n.v[q].is_sym("declare-type")) b.declare = truthy(n.v[q + 1]);
        else if (n.v[q].is_sym("reduction")) b.reduction = truthy(n.v[q + 1]);
        else if (n.v[q].is_sym("grid")) {
          const Sx &g = n.v[q + 1];
          if (!g.is_list() || g.n() != 3 || g.v[0].kind != Sx::INT || g.v[0].i < 0 || g.v[0].i > 2)
            return err = "expr: :grid (RANK GLOBAL-SIZE LOCAL-SIZE) with rank 0, 1 or 2", false;
          b.grid_rank = (int)g.v[0].i;
          b.grid_global = g.v[1];
          b.grid_local = g.v[2];
        }
      }
      if (b.writes.empty()) return err = "expr: no write", false;
      if (!cdtypes().count(b.dtype)) return err = "expr: unknown dtype " + b.dtype, false;
      it.body.push_back(b);
    } else {
      return err = "unknown blueprint node :" + ty, false;
    }
  }
  if (depth || ifs) return err = "unbalanced for / if", false;
  return true;
}

// ------------------------------------------------------------------ expressions -> HIP
struct Rend {
  std::string err;

  static std::string fmt_float(double v, bool f64) {
    if (isinf(v)) return v > 0 ? "_infinity" : "_negative_infinity";
    if (isnan(v)) return "_nan";
    char buf[64];
    if (f64) {
      snprintf(buf, sizeof(buf), "%.17g", v);
      std::string s = buf;
      if (s.find('.') == std::string::npos && s.find('e') == std::string::npos) s += ".0";
      return s;
    }
    // the shortest decimal that reads back as the same float, in positional notation (as Caten's ~f prints)
    const float fv = (float)v;
    if (isinf(fv)) return fv > 0 ? "_infinity" : "_negative_infinity";  // a double past the float range
    int prec = 0;
    for (; prec <= 8; prec++) {
      snprintf(buf, sizeof(buf), "%.*e", prec, (double)fv);
      if (strtof(buf, nullptr) == fv) break;
    }
    std::string m = buf;  // [-]d.ddde[+-]xx
    const bool negative = m[0] == '-';
    if (negative) m = m.substr(1);
    const size_t ep = m.find('e');
    const int ex = atoi(m.c_str() + ep + 1);
    std::string digits;
    for (size_t k = 0; k < ep; k++)
      if (m[k] != '.') digits.push_back(m[k]);
    while (digits.size() > 1 && digits.back() == '0') digits.pop_back();
    std::string s;
    if (ex >= 0) {
      while ((int)digits.size() < ex + 1) digits.push_back('0');
      s = digits.substr(0, (size_t)ex + 1) + "." + ((int)digits.size() > ex + 1 ? digits.substr((size_t)ex + 1) : "0");
    } else {
      s = "0." + std::string((size_t)(-ex - 1), '0') + digits;
    }
    return (negative ? "-" : "") + s + "f";
  }

  // %render-const (renderer.lisp:319-329)
  std::string constant(const Sx &v, const std::string &dtype) {
    if (v.is_sym("t")) return "true";
    if (v.is_sym("nil")) return "false";
    const bool fl = dtype.rfind("float", 0) == 0;
    if (v.kind == Sx::FLT || (fl && v.kind == Sx::INT)) return fmt_float(v.kind == Sx::FLT ? v.f : (double)v.i, dtype == "float64");
    if (v.kind == Sx::INT) return std::to_string(v.i);
    if (v.kind == Sx::SYM) return v.s;
    err = "cannot render a constant";
    return "0";
  }

  // element reads that the kernel holds in registers: the rendered reference -> the register that has it
  std::map<std::string, std::string> held;

  std::string aref(const Sx &e) {
    if (e.n() < 2) { err = "(aref ID [INDEX])"; return "0"; }
    const std::string &name = e.v[1].s;
    if (e.n() == 2 || e.v[2].is_sym("nil")) return name;
    const std::string ref = name + "[" + expr(e.v[2], "int64") + "]";
    auto h = held.find(ref);
    return h == held.end() ? ref : h->second;
  }

  // render-expr / %render-node dispatch (renderer.lisp:331-411)
  std::string expr(const Sx &e, const std::string &fd) {
    if (e.kind == Sx::INT) return std::to_string(e.i);
    if (e.kind == Sx::FLT) return fmt_float(e.f, fd == "float64");
    if (e.kind == Sx::SYM) return e.is_sym("t") ? "true" : e.is_sym("nil") ? "false" : e.s;
    if (e.kind == Sx::STR) return e.s;
    if (e.v.empty() || e.v[0].kind != Sx::SYM) { err = "an expression must be headed by its operation"; return "0"; }
    const std::string &op = e.v[0].s;
    const bool f64 = fd == "float64";
    auto r = [&](size_t k) { return expr(e.v[k], fd); };
    const size_t na = e.n() - 1;
    auto need = [&](size_t k) {
      if (na < k) { err = "too few arguments for :" + op; return false; }
      return true;
    };
    if (op == "const") return need(1) ? constant(e.v[1], na >= 2 ? e.v[2].s : fd) : "0";
    if (op == "aref") return aref(e);
    if (op == "space") {  // metal.lisp:173-176 -> blockIdx / threadIdx
      if (!need(2)) return "0";
      const char *xyz[3] = {"x", "y", "z"};
      const long long rank = e.v[2].i;
      if (rank < 0 || rank > 2) { err = "space: rank is 0, 1 or 2"; return "0"; }
      return std::string(e.v[1].is_sym("block") ? "blockIdx." : "threadIdx.") + xyz[rank];
    }
    static const std::map<std::string, std::string> infix = {{"add", "+"}, {"mul", "*"}, {"mod", "%"}, {"idiv", "/"}, {"and", " & "}, {"or", " | "}, {"xor", " ^ "}};
    auto inf = infix.find(op);
    if (inf != infix.end()) {
      if (!need(1)) return "0";
      std::string s = "(";
      for (size_t k = 1; k <= na; k++) s += (k > 1 ? inf->second : "") + r(k);
      return s + ")";
    }
    if (op == "wmma") return need(3) ? "(" + r(1) + "+" + r(2) + "*" + r(3) + ")" : "0";
    if (op == "max") return need(2) ? "ct_max(" + r(1) + ", " + r(2) + ")" : "0";
    if (op == "neg") return need(1) ? "(-" + r(1) + ")" : "0";
    if (op == "not") return need(1) ? "(!" + r(1) + ")" : "0";
    if (op == "sin" || op == "log2" || op == "exp2" || op == "sqrt") return need(1) ? op + (f64 ? "" : "f") + "(" + r(1) + ")" : "0";
    if (op == "recip") {
      if (!need(1)) return "0";
      if (fd.rfind("float", 0) == 0) return std::string(f64 ? "(1.0" : "(1.0f") + "/(" + r(1) + "))";
      return "(1/(" + r(1) + "))";
    }
    if (op == "!=" || op == "<") return need(2) ? "(" + r(na - 1) + op + r(na) + ")" : "0";
    if (op == "move" || op == "store") return need(1) ? r(na) : "0";
    if (op == "cast") {
      if (!need(2)) return "0";
      auto ct = cdtypes().find(e.v[1].s);
      if (ct == cdtypes().end()) { err = "cast: unknown dtype " + e.v[1].s; return "0"; }
      return "((" + ct->second + ")" + r(na) + ")";
    }
    if (op == "where") return need(3) ? "(" + r(1) + " ? " + r(2) + " : " + r(3) + ")" : "0";
    err = "Hip-Renderer: no %render-node method for :" + op;
    return "0";
  }
};

static bool uses(const Sx &e, const std::string &sym) {
  if (e.kind == Sx::SYM) return e.s == sym;
  if (e.kind != Sx::LIST) return false;
  for (size_t k = (e.call("aref") || e.call("cast") || e.call("const")) ? 1 : 0; k < e.n(); k++)
    if (uses(e.v[k], sym)) return true;
  return false;
}
static bool is_scalar_ref(const Sx &w) { return w.kind == Sx::SYM || (w.call("aref") && (w.n() == 2 || w.v[2].is_sym("nil"))); }
static std::string ref_name(const Sx &w) { return w.kind == Sx::SYM ? w.s : (w.call("aref") && w.n() >= 2 ? w.v[1].s : std::string()); }
static bool const_value(const Sx &e, double &out) {
  if (e.kind == Sx::INT) { out = (double)e.i; return true; }
  if (e.kind == Sx::FLT) { out = e.f; return true; }
  if (e.call("const") && e.n() >= 2) return const_value(e.v[1], out);
  if (e.call("neg") && e.n() == 2 && const_value(e.v[1], out)) { out = -out; return true; }
  return false;
}
static bool is_zero(const Sx &e) {
  double v;
  return const_value(e, v) && v == 0.0;
}
static bool is_one(const Sx &e) {
  double v;
  return const_value(e, v) && v == 1.0;
}
// `below` is the condition (idx < N); returns N when it has that shape and by == 1
static const Sx *upper_bound(const BpNode &f) {
  if (!is_one(f.by)) return nullptr;
  if (f.below.call("<") && f.below.n() >= 3) {
    const Sx &x = f.below.v[f.below.n() - 2], &y = f.below.v[f.below.n() - 1];
    if (x.kind == Sx::SYM && x.s == f.idx) return &y;
  }
  return nullptr;
}
static int match_end(const std::vector<BpNode> &b, int i) {  // index of the ENDFOR that closes the FOR at i
  int lvl = 0;
  for (int j = i; j < (int)b.size(); j++) {
    if (b[j].t == BpNode::FOR) lvl++;
    else if (b[j].t == BpNode::ENDFOR && --lvl == 0) return j;
  }
  return -1;
}

// Expressions over the by-value arguments (grid sizes, route shapes), evaluated on the host.  Integer arithmetic is
// exact (loop bounds, strides); the float instructions cover how the GLOBAL directive spells a grid size,
// cast_int(ceil-ish(float(upper - from) / float(by)) / local-size) (directive.lisp:97-100).
static bool eval_num(const Sx &e, const std::map<std::string, long long> &env, double &out, bool &is_int) {
  if (e.kind == Sx::INT) { out = (double)e.i; is_int = true; return true; }
  if (e.kind == Sx::FLT) { out = e.f; is_int = false; return true; }
  if (e.kind == Sx::SYM) {
    auto it = env.find(e.s);
    if (it == env.end()) return false;
    out = (double)it->second;
    is_int = true;
    return true;
  }
  if (e.kind != Sx::LIST || e.v.empty() || e.v[0].kind != Sx::SYM) return false;
  const std::string &op = e.v[0].s;
  if (op == "const") {
    if (e.n() < 2 || !eval_num(e.v[1], env, out, is_int)) return false;
    if (e.n() >= 3 && e.v[2].kind == Sx::SYM && e.v[2].s.rfind("float", 0) == 0) is_int = false;
    return true;
  }
  if (op == "cast") {
    if (e.n() < 3 || !eval_num(e.v[e.n() - 1], env, out, is_int)) return false;
    const bool to_float = e.v[1].kind == Sx::SYM && e.v[1].s.rfind("float", 0) == 0;
    if (!to_float) out = trunc(out);  // a C cast to an integer type
    is_int = !to_float;
    return true;
  }
  std::vector<double> a;
  bool all_int = true;
  for (size_t k = 1; k < e.n(); k++) {
    if (e.v[k].is_sym("nil")) continue;  // the placeholder read of :< / :!=
    double v;
    bool vi;
    if (!eval_num(e.v[k], env, v, vi)) return false;
    a.push_back(v);
    all_int = all_int && vi;
  }
  if (a.empty()) return false;
  is_int = all_int;
  if (op == "add") { out = 0; for (double v : a) out += v; return true; }
  if (op == "mul") { out = 1; for (double v : a) out *= v; return true; }
  if (op == "neg") { out = -a[0]; return true; }
  if (op == "max" && a.size() == 2) { out = a[0] > a[1] ? a[0] : a[1]; return true; }
  if (op == "recip") {
    if (a[0] == 0) return false;
    if (all_int) out = trunc(1.0 / a[0]);
    else out = 1.0 / a[0];
    return true;
  }
  if (op == "idiv" && a.size() == 2 && a[1] != 0) { out = all_int ? trunc(a[0] / a[1]) : a[0] / a[1]; return true; }
  if (op == "mod" && a.size() == 2 && a[1] != 0 && all_int) { out = (double)((long long)a[0] % (long long)a[1]); return true; }
  if (op == "move" || op == "store") { out = a.back(); return true; }
  return false;
}
static bool eval_int(const Sx &e, const std::map<std::string, long long> &env, long long &out) {
  double v;
  bool is_int;
  if (!eval_num(e, env, v, is_int) || v != trunc(v) || fabs(v) > 9e15) return false;
  out = (long long)v;
  return true;
}

// ------------------------------------------------------------------ routes to hand-written kernels
// An index expression as an affine function of (up to three) loop indices, found by evaluation: base and one
// coefficient per index, confirmed on a probe point.  Whatever way the scheduler spelled the index, a matrix
// laid out row-major gives the same numbers.
struct Affine {
  long long base = 0, c[3] = {0, 0, 0};
};
static bool affine_of(const Sx &index, const std::string idx[3], int nidx, std::map<std::string, long long> env, Affine &out) {
  auto at = [&](long long a, long long b, long long c, long long &v) {
    const long long p[3] = {a, b, c};
    for (int k = 0; k < nidx; k++) env[idx[k]] = p[k];
    return eval_int(index, env, v);
  };
  long long v0, v;
  if (!at(0, 0, 0, v0)) return false;
  out.base = v0;
  for (int k = 0; k < nidx; k++) {
    if (!at(k == 0, k == 1, k == 2, v)) return false;
    out.c[k] = v - v0;
  }
  if (!at(2, 3, 5, v)) return false;
  return v == v0 + 2 * out.c[0] + (nidx > 1 ? 3 * out.c[1] : 0) + (nidx > 2 ? 5 * out.c[2] : 0);
}

// the same over any number of indices
struct AffineN {
  long long base = 0;
  std::vector<long long> c;
};
static bool affine_n(const Sx &index, const std::vector<std::string> &idx, std::map<std::string, long long> env, AffineN &out) {
  const int n = (int)idx.size();
  auto at = [&](int unit, bool check, long long &v) {
    for (int k = 0; k < n; k++) env[idx[k]] = check ? 2 + 3 * k : (k == unit ? 1 : 0);
    return eval_int(index, env, v);
  };
  long long v0, v;
  if (!at(-1, false, v0)) return false;
  out.base = v0;
  out.c.assign(n, 0);
  for (int k = 0; k < n; k++) {
    if (!at(k, false, v)) return false;
    out.c[k] = v - v0;
  }
  if (!at(-1, true, v)) return false;
  long long want = v0;
  for (int k = 0; k < n; k++) want += (2 + 3 * k) * out.c[k];
  return v == want;
}

enum RouteKind { R_NONE = 0, R_MATMUL, R_EMBEDDING, R_ARGMAX, R_SOFTMAX, R_LAYERNORM, R_RMSNORM };
struct Route {
  RouteKind kind = R_NONE;
  int out = -1, a = -1, b = -1, bias = -1;  // argument positions
  Sx out_idx, a_idx, b_idx, bias_idx;       // index expressions over the loop indices
  std::string idx[3];                       // loop indices: (i, j, k) / (t, d, v) / (row, col)
  Sx bound[3];                              // their upper bounds
  int act = CTHIP_ACT_NONE;
  double eps = 0.0;                         // LayerNorm / RMSNorm: read off the item by evaluation
  // matmul: the parallel loops outermost first (batch..., row i, column j), then the reduction index k
  std::vector<std::string> lidx;
  std::vector<Sx> lbound;
  // matmul epilogue act(alpha * acc + pre...) + post...: up to two more operands, each added before or after the
  // activation; embedding: the addend of `acc + other[..]`
  int extra[2] = {-1, -1};
  Sx extra_idx[2];
  bool extra_post[2] = {false, false};
  double alpha = 1.0;
};

struct Program {
  Item item;
  std::string source, route_name = "rendered", last_route = "none";
  std::vector<Sx> grid_bounds;
  int rows_per_block = 256;
  bool parallel = false;
  bool explicit_grid = false;  // the blueprint carries its own launch sizes (ExprGrid)
  Sx grid_global[3], grid_local[3];
  Route route;
  hipFunction_t fn = nullptr;
  // what the matmul route derived from the shape arguments at the last launch: the layers of a model share one program
  // and launch it with the same shapes, so the index expressions are evaluated once per set of values
  std::vector<long long> memo_key, memo_ext;
  bool memo_ok = false;
  AffineN memo_aff[5];
};

static int arg_pos(const Item &it, const std::string &id) {
  for (size_t k = 0; k < it.globals.size(); k++)
    if (it.globals[k].id == id) return (int)k;
  return -1;
}
static bool is_ref_to(const Sx &e, const std::string &name) { return is_scalar_ref(e) && ref_name(e) == name; }

// acc = acc + X  /  acc = X + acc  /  (wmma acc a b); returns X (for wmma: (mul a b))
static bool reduction_term(const BpNode &n, const std::string &acc, const char *op, Sx &term) {
  if (n.t != BpNode::EXPR || n.writes.size() != 1 || !is_ref_to(n.writes[0], acc)) return false;
  const Sx &e = n.rhs;
  if (!strcmp(op, "add") && e.call("wmma") && e.n() == 4 && is_ref_to(e.v[1], acc)) {
    term = sx_list({sx_sym("mul"), e.v[2], e.v[3]});
    return true;
  }
  if (!e.call(op) || e.n() != 3) return false;
  if (is_ref_to(e.v[1], acc) && !uses(e.v[2], acc)) { term = e.v[2]; return true; }
  if (is_ref_to(e.v[2], acc) && !uses(e.v[1], acc)) { term = e.v[1]; return true; }
  return false;
}
static bool is_global_aref(const Item &it, const Sx &e, int &pos) {
  if (!e.call("aref") || e.n() < 3) return false;
  pos = arg_pos(it, e.v[1].s);
  return pos >= 0 && it.globals[pos].pointer && it.globals[pos].dtype == "float32";
}

// ---- recognition by VALUE ----
// The scalar statements between the loops (mean = s / n, rstd = 1 / sqrt(q / n + eps)) and the per-element
// expressions come in whatever spelling the simplifier left (recip of a cast, a folded constant, operands in any
// order), so they are recognised by VALUE: evaluated on probe numbers and compared with what the norm computes.
struct Probe {
  const Item *it = nullptr;
  std::map<std::string, double> scalars;  // temporaries and by-value arguments
  std::map<int, double> arrays;           // argument position of a global array -> what any element of it reads as
  std::map<int, Sx> index;                // the index expression each array was read with
};
static bool sx_equal(const Sx &a, const Sx &b) {
  if (a.kind != b.kind) return false;
  if (a.kind == Sx::LIST) {
    if (a.n() != b.n()) return false;
    for (size_t k = 0; k < a.n(); k++)
      if (!sx_equal(a.v[k], b.v[k])) return false;
    return true;
  }
  return a.s == b.s && a.i == b.i && a.f == b.f;
}
static bool probe(const Sx &e, Probe &p, double &out) {
  if (e.kind == Sx::INT) { out = (double)e.i; return true; }
  if (e.kind == Sx::FLT) { out = e.f; return true; }
  if (e.kind == Sx::SYM) {
    auto f = p.scalars.find(e.s);
    if (f == p.scalars.end()) return false;
    out = f->second;
    return true;
  }
  if (e.kind != Sx::LIST || e.v.empty() || e.v[0].kind != Sx::SYM) return false;
  const std::string &op = e.v[0].s;
  if (op == "aref") {
    if (is_scalar_ref(e)) {
      auto f = p.scalars.find(ref_name(e));
      if (f == p.scalars.end()) return false;
      out = f->second;
      return true;
    }
    int pos;
    if (!is_global_aref(*p.it, e, pos)) return false;
    auto f = p.arrays.find(pos);
    if (f == p.arrays.end()) return false;
    auto seen = p.index.find(pos);
    if (seen == p.index.end()) p.index[pos] = e.v[2];
    else if (!sx_equal(seen->second, e.v[2])) return false;  // one element of each array per iteration
    out = f->second;
    return true;
  }
  if (op == "const") return e.n() >= 2 && probe(e.v[1], p, out);
  if (op == "cast") {
    if (e.n() < 3 || e.v[1].kind != Sx::SYM || e.v[1].s.rfind("float", 0) != 0) return false;
    return probe(e.v[e.n() - 1], p, out);
  }
  std::vector<double> a;
  for (size_t k = 1; k < e.n(); k++) {
    double v;
    if (!probe(e.v[k], p, v)) return false;
    a.push_back(v);
  }
  if (a.empty()) return false;
  if (op == "add") { out = 0; for (double v : a) out += v; return true; }
  if (op == "mul") { out = 1; for (double v : a) out *= v; return true; }
  if (op == "neg" && a.size() == 1) { out = -a[0]; return true; }
  if (op == "recip" && a.size() == 1 && a[0] != 0) { out = 1.0 / a[0]; return true; }
  if (op == "sqrt" && a.size() == 1 && a[0] >= 0) { out = sqrt(a[0]); return true; }
  if (op == "max" && a.size() == 2) { out = a[0] > a[1] ? a[0] : a[1]; return true; }
  if (op == "exp2" && a.size() == 1) { out = exp2(a[0]); return true; }
  return false;
}
// (1e-6: a shape that is static lets the simplifier fold 1 / n into a single-float constant, 3e-8 off)
static bool near(double a, double b) { return fabs(a - b) <= 1e-6 * (1.0 + fabs(b)); }
static void global_arefs(const Item &it, const Sx &e, std::vector<int> &out) {
  int pos;
  if (e.call("aref")) {
    if (is_global_aref(it, e, pos) && std::find(out.begin(), out.end(), pos) == out.end()) out.push_back(pos);
    return;
  }
  if (e.kind == Sx::LIST)
    for (const Sx &c : e.v) global_arefs(it, c, out);
}

// what the activations of the hand-written kernels compute, in double (Caten's decompositions: tanh(y) = 2 sigmoid(2y) - 1,
// sigmoid(z) = recip(1 + exp2(-z / ln 2)); nn/activations.lisp:3-7,180-215, api/high-level-ops.lisp:112-117)
static double act_value(int act, double x) {
  switch (act) {
    case CTHIP_ACT_RELU: return x > 0 ? x : 0.0;
    case CTHIP_ACT_GELU: return 0.5 * x * (1.0 + tanh(0.7978845608028654 * (x + 0.044715 * x * x * x)));
    case CTHIP_ACT_SILU: return x / (1.0 + exp(-x));
    case CTHIP_ACT_SIGMOID: return 1.0 / (1.0 + exp(-x));
    case CTHIP_ACT_TANH: return tanh(x);
    default: return x;
  }
}

// The statement that stores a matmul's result, recognised by VALUE: with the accumulator and the (up to two) other
// arrays it reads set to probe numbers it has to give act(alpha * acc + pre...) + post... for one of the kernels'
// activations and one assignment of the arrays to "before" / "after" the activation.  Without an activation any
// factor alpha is accepted (attention's scores * recip(sqrt(head-dim)), external/llm/layers.lisp:3-5), with one
// alpha is 1 (GELU after c_fc, ReLU: source/test-suite/test-scheduler.lisp:140-163).
static bool probe_matmul_epilogue(const Item &it, const Sx &rhs, const std::string &acc, Route &r) {
  std::vector<int> arrs;
  global_arefs(it, rhs, arrs);
  if (arrs.size() > 2) return false;
  for (int a : arrs)
    if (a == r.out) return false;
  Probe p;
  p.it = &it;
  auto f = [&](double a, double e0, double e1, double &out) {
    p.arrays.clear();
    p.index.clear();
    p.scalars[acc] = a;
    if (arrs.size() > 0) p.arrays[arrs[0]] = e0;
    if (arrs.size() > 1) p.arrays[arrs[1]] = e1;
    return probe(rhs, p, out);
  };
  auto loose = [](double a, double b) { return fabs(a - b) <= 1e-5 * (1.0 + fabs(b)); };  // float-rounded GELU constants
  const double pts[4][3] = {{0.7, 0.3, -0.2}, {-1.3, 0.5, 1.1}, {2.1, -0.4, 0.6}, {-0.15, -0.05, 0.1}};
  double v0, v1;
  if (!f(0.0, 0.0, 0.0, v0) || !f(1.0, 0.0, 0.0, v1)) return false;
  const int acts[6] = {CTHIP_ACT_NONE, CTHIP_ACT_RELU, CTHIP_ACT_GELU, CTHIP_ACT_SILU, CTHIP_ACT_SIGMOID, CTHIP_ACT_TANH};
  for (int act : acts) {
    const double alpha = act == CTHIP_ACT_NONE ? v1 - v0 : 1.0;
    if (act == CTHIP_ACT_NONE && (v0 != 0.0 || alpha == 0.0 || !std::isfinite(alpha))) continue;
    for (int roles = 0; roles < (act == CTHIP_ACT_NONE ? 1 : 1 << arrs.size()); roles++) {
      bool ok = true;
      for (int q = 0; q < 4 && ok; q++) {
        double got;
        if (!f(pts[q][0], pts[q][1], pts[q][2], got)) return false;
        double pre = alpha * pts[q][0], post = 0.0;
        for (size_t k = 0; k < arrs.size(); k++) ((roles >> k) & 1 ? post : pre) += pts[q][1 + k];
        ok = loose(got, act_value(act, pre) + post);
      }
      if (!ok) continue;
      r.act = act;
      r.alpha = alpha;
      for (size_t k = 0; k < arrs.size(); k++) {
        r.extra[k] = arrs[k];
        r.extra_idx[k] = p.index[arrs[k]];
        r.extra_post[k] = (roles >> k) & 1;
      }
      return true;
    }
  }
  return false;
}

// for (batch...): for i < M: for j < N: { acc = 0; for k < K: acc += A[..] * B[..]; out[..] = epilogue(acc) }
// -- the nest of (caten (!matmul a b)), with up to three batch loops in front (source/test-suite/test-scheduler.lisp:126-138)
static bool match_matmul(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  const int n = (int)b.size();
  if (n < 9 || (n - 5) % 2) return false;
  const int P = (n - 5) / 2;  // parallel loops
  if (P < 2 || P > 5) return false;
  for (int q = 0; q < P; q++)
    if (b[q].t != BpNode::FOR || b[n - 1 - q].t != BpNode::ENDFOR) return false;
  if (b[P].t != BpNode::EXPR || b[P + 1].t != BpNode::FOR || b[P + 2].t != BpNode::EXPR || b[P + 3].t != BpNode::ENDFOR || b[P + 4].t != BpNode::EXPR)
    return false;
  for (int q = 0; q <= P; q++) {
    const BpNode &f = b[q < P ? q : P + 1];
    const Sx *ub = upper_bound(f);
    if (!ub || !is_zero(f.upfrom)) return false;
    r.lidx.push_back(f.idx);
    r.lbound.push_back(*ub);
  }
  const BpNode &decl = b[P], &red = b[P + 2], &st = b[P + 4];
  if (!decl.declare || decl.writes.size() != 1 || !is_scalar_ref(decl.writes[0]) || !is_zero(decl.rhs) || decl.dtype != "float32") return false;
  const std::string acc = ref_name(decl.writes[0]);
  Sx term;
  if (!reduction_term(red, acc, "add", term) || !term.call("mul") || term.n() != 3) return false;
  if (!is_global_aref(it, term.v[1], r.a) || !is_global_aref(it, term.v[2], r.b)) return false;
  r.a_idx = term.v[1].v[2];
  r.b_idx = term.v[2].v[2];
  if (st.writes.size() != 1 || !is_global_aref(it, st.writes[0], r.out) || it.globals[r.out].type != "output") return false;
  r.out_idx = st.writes[0].v[2];
  if (r.out == r.a || r.out == r.b) return false;
  if (!probe_matmul_epilogue(it, st.rhs, acc, r)) return false;
  r.kind = R_MATMUL;
  return true;
}

// for t < T: for d < D: { acc = 0; for v < V: acc += where(eq(v, idx[t]), W[v, d], 0); out[t, d] = acc }
// (eq is spelled not(!=), source/api/function.lisp; the compared index may be cast to the table's dtype)
static const Sx &strip_cast(const Sx &e) { return (e.call("cast") && e.n() == 3) ? strip_cast(e.v[2]) : e; }
static bool match_embedding(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  if (b.size() != 9) return false;
  if (b[0].t != BpNode::FOR || b[1].t != BpNode::FOR || b[2].t != BpNode::EXPR || b[3].t != BpNode::FOR || b[4].t != BpNode::EXPR ||
      b[5].t != BpNode::ENDFOR || b[6].t != BpNode::EXPR || b[7].t != BpNode::ENDFOR || b[8].t != BpNode::ENDFOR)
    return false;
  const int fors[3] = {0, 1, 3};
  for (int q = 0; q < 3; q++) {
    const Sx *ub = upper_bound(b[fors[q]]);
    if (!ub || !is_zero(b[fors[q]].upfrom)) return false;
    r.idx[q] = b[fors[q]].idx;
    r.bound[q] = *ub;
  }
  if (!b[2].declare || b[2].writes.size() != 1 || !is_scalar_ref(b[2].writes[0]) || !is_zero(b[2].rhs)) return false;
  const std::string acc = ref_name(b[2].writes[0]);
  Sx term;
  if (!reduction_term(b[4], acc, "add", term) || !term.call("where") || term.n() != 4 || !is_zero(term.v[3])) return false;
  const Sx &cond = term.v[1];
  if (!cond.call("not") || cond.n() != 2 || !cond.v[1].call("!=") || cond.v[1].n() < 3) return false;
  const Sx &x = strip_cast(cond.v[1].v[cond.v[1].n() - 2]), &y = strip_cast(cond.v[1].v[cond.v[1].n() - 1]);
  // one side is the vocabulary index (any spelling of it, checked by evaluation at launch), the other the token
  // id read from the input
  const Sx *vside = nullptr, *tside = nullptr;
  int dummy;
  if (uses(x, r.idx[2]) && !is_global_aref(it, x, dummy)) vside = &x, tside = &y;
  else if (uses(y, r.idx[2]) && !is_global_aref(it, y, dummy)) vside = &y, tside = &x;
  if (!vside) return false;
  if (is_global_aref(it, *tside, r.b)) {
    if (uses(tside->v[2], r.idx[2]) || uses(tside->v[2], r.idx[1])) return false;
    r.b_idx = tside->v[2];
  } else {
    // the row is an EXPRESSION of the token position, not a stored index: wpe(start-pos + arange(seq-len)) of
    // Transformer (external/llm/layers.lisp:81); which rows it names is worked out at launch
    if (uses(*tside, r.idx[2]) || uses(*tside, r.idx[1]) || !uses(*tside, r.idx[0])) return false;
    std::vector<int> none;
    global_arefs(it, *tside, none);
    if (!none.empty()) return false;
    r.b = -1;
    r.b_idx = *tside;
  }
  r.bias_idx = *vside;
  if (!is_global_aref(it, term.v[2], r.a)) return false;
  r.a_idx = term.v[2].v[2];
  if (b[6].writes.size() != 1 || !is_global_aref(it, b[6].writes[0], r.out)) return false;
  r.out_idx = b[6].writes[0].v[2];
  // the stored value: acc, or acc + other[..] (the sum of two embeddings, layers.lisp:82)
  const Sx &e = b[6].rhs;
  if (!is_ref_to(e, acc)) {
    if (!e.call("add") || e.n() != 3) return false;
    const int ai = is_ref_to(e.v[1], acc) ? 1 : is_ref_to(e.v[2], acc) ? 2 : 0;
    if (!ai || !is_global_aref(it, e.v[3 - ai], r.extra[0]) || r.extra[0] == r.out) return false;
    r.extra_idx[0] = e.v[3 - ai].v[2];
  }
  r.kind = R_EMBEDDING;
  return true;
}

// for r < R: { m = -inf; for i < N: m = max(m, x[r, i]); g = 0; for i < N: g = max(g, where(eq(x[r, i], m), (N - 1) - i, 0));
//              out[r] = cast(N - g - 1) }      -- ArgMaxNode, lowest index among ties
static bool match_argmax(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  if (b.size() != 11) return false;
  const BpNode::T want[11] = {BpNode::FOR, BpNode::EXPR, BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR, BpNode::FOR,
                              BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR, BpNode::ENDFOR};
  for (int k = 0; k < 11; k++)
    if (b[k].t != want[k]) return false;
  const Sx *rows = upper_bound(b[0]), *n1 = upper_bound(b[2]), *n2 = upper_bound(b[6]);
  if (!rows || !n1 || !n2 || !is_zero(b[0].upfrom) || !is_zero(b[2].upfrom) || !is_zero(b[6].upfrom)) return false;
  r.idx[0] = b[0].idx;
  r.idx[1] = b[2].idx;
  r.bound[0] = *rows;
  r.bound[1] = *n1;
  double v;
  if (!b[1].declare || !const_value(b[1].rhs, v) || !(isinf(v) && v < 0) || !is_scalar_ref(b[1].writes[0])) return false;
  const std::string m = ref_name(b[1].writes[0]);
  Sx term;
  if (!reduction_term(b[3], m, "max", term) || !is_global_aref(it, term, r.a)) return false;
  r.a_idx = term.v[2];
  if (!b[5].declare || !is_zero(b[5].rhs) || !is_scalar_ref(b[5].writes[0])) return false;
  const std::string g = ref_name(b[5].writes[0]);
  Sx t2;
  if (!reduction_term(b[7], g, "max", t2) || !t2.call("where") || t2.n() != 4 || !is_zero(t2.v[3])) return false;
  const Sx &cond = t2.v[1];
  if (!cond.call("not") || cond.n() != 2 || !cond.v[1].call("!=") || cond.v[1].n() < 3) return false;
  const Sx &x = cond.v[1].v[cond.v[1].n() - 2], &y = cond.v[1].v[cond.v[1].n() - 1];
  int xa = -1;
  if (!((is_global_aref(it, x, xa) && is_ref_to(y, m)) || (is_global_aref(it, y, xa) && is_ref_to(x, m))) || xa != r.a) return false;
  // the value kept is (N - 1) - i, in any spelling: checked by evaluation at launch
  r.b_idx = strip_cast(t2.v[2]);
  if (b[6].idx != r.idx[1]) r.idx[2] = b[6].idx;  // the second loop's own index name: evaluation binds both
  int op = -1;
  if (b[9].writes.size() != 1 || !b[9].writes[0].call("aref") || (op = arg_pos(it, b[9].writes[0].v[1].s)) < 0) return false;
  if (it.globals[op].dtype != "int64" || !it.globals[op].pointer) return false;
  r.out = op;
  r.out_idx = b[9].writes[0].n() > 2 ? b[9].writes[0].v[2] : sx_int(0);
  r.bias_idx = strip_cast(b[9].rhs);  // N - g - 1, checked by evaluation at launch
  r.idx[2] = r.idx[2].empty() ? r.idx[1] : r.idx[2];
  r.kind = R_ARGMAX;
  r.bound[2] = sx_sym(g);  // the name of the kept maximum: the launch evaluates the final expression over it
  return true;
}

// for r < R: { m = -inf; for i: m = max(m, x); s = 0; for i: s += exp2((x - m) * c); for i: y = exp2((x - m) * c) * recip(s) }
static bool is_exp_of_shifted(const Item &it, const Sx &e, const std::string &m, int &xpos, Sx &xidx) {
  if (!e.call("exp2") || e.n() != 2) return false;
  const Sx &mul = e.v[1];
  if (!mul.call("mul") || mul.n() != 3) return false;
  double c;
  const Sx *sh = nullptr;
  if (const_value(mul.v[2], c)) sh = &mul.v[1];
  else if (const_value(mul.v[1], c)) sh = &mul.v[2];
  if (!sh || fabs(c - 1.4426950408889634) > 1e-5) return false;
  if (!sh->call("add") || sh->n() != 3) return false;
  const Sx *xa = nullptr, *neg = nullptr;
  if (sh->v[2].call("neg")) xa = &sh->v[1], neg = &sh->v[2];
  else if (sh->v[1].call("neg")) xa = &sh->v[2], neg = &sh->v[1];
  if (!xa || neg->n() != 2 || !is_ref_to(neg->v[1], m) || !is_global_aref(it, *xa, xpos)) return false;
  xidx = xa->v[2];
  return true;
}
static bool match_softmax(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  if (b.size() != 13) return false;
  const BpNode::T want[13] = {BpNode::FOR, BpNode::EXPR, BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR, BpNode::FOR,
                              BpNode::EXPR, BpNode::ENDFOR, BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::ENDFOR};
  for (int k = 0; k < 13; k++)
    if (b[k].t != want[k]) return false;
  const Sx *rows = upper_bound(b[0]), *n1 = upper_bound(b[2]), *n2 = upper_bound(b[6]), *n3 = upper_bound(b[9]);
  if (!rows || !n1 || !n2 || !n3 || !is_zero(b[0].upfrom) || !is_zero(b[2].upfrom) || !is_zero(b[6].upfrom) || !is_zero(b[9].upfrom)) return false;
  if (b[2].idx != b[6].idx || b[2].idx != b[9].idx) return false;
  r.idx[0] = b[0].idx;
  r.idx[1] = b[2].idx;
  r.bound[0] = *rows;
  r.bound[1] = *n1;
  double v;
  if (!b[1].declare || !const_value(b[1].rhs, v) || !(isinf(v) && v < 0) || !is_scalar_ref(b[1].writes[0])) return false;
  const std::string m = ref_name(b[1].writes[0]);
  Sx term;
  if (!reduction_term(b[3], m, "max", term) || !is_global_aref(it, term, r.a)) return false;
  r.a_idx = term.v[2];
  if (!b[5].declare || !is_zero(b[5].rhs) || !is_scalar_ref(b[5].writes[0])) return false;
  const std::string s = ref_name(b[5].writes[0]);
  Sx t2, xi;
  int xp = -1;
  if (!reduction_term(b[7], s, "add", t2) || !is_exp_of_shifted(it, t2, m, xp, xi) || xp != r.a || !sx_equal(xi, r.a_idx)) return false;
  const Sx &e = b[10].rhs;
  if (!e.call("mul") || e.n() != 3) return false;
  const Sx *ex = nullptr, *rc = nullptr;
  if (e.v[2].call("recip")) ex = &e.v[1], rc = &e.v[2];
  else if (e.v[1].call("recip")) ex = &e.v[2], rc = &e.v[1];
  if (!ex || rc->n() != 2 || !is_ref_to(rc->v[1], s) || !is_exp_of_shifted(it, *ex, m, xp, xi) || xp != r.a || !sx_equal(xi, r.a_idx)) return false;
  if (b[10].writes.size() != 1 || !is_global_aref(it, b[10].writes[0], r.out) || r.out == r.a) return false;
  r.out_idx = b[10].writes[0].v[2];
  r.kind = R_SOFTMAX;
  return true;
}

// ---- LayerNorm / RMSNorm rows (source/nn/normalization.lisp:39-58,78-92) ----
// the row length as the probes see it: a literal bound is itself, a symbolic one is bound to 7
static bool probe_row_length(const Sx &bound, Probe &p, double &n) {
  if (const_value(bound, n)) return n >= 1;
  if (bound.kind != Sx::SYM) return false;
  p.scalars[bound.s] = n = 7.0;
  return true;
}
// rr = 1 / sqrt(q / n + eps): eps is what the statement gives at q = 0, confirmed at a second point
static bool probe_rstd(const BpNode &st, const std::string &q, Probe &p, double n, double &eps) {
  if (st.t != BpNode::EXPR || !st.declare || st.writes.size() != 1 || !is_scalar_ref(st.writes[0])) return false;
  double v0, v1;
  p.scalars[q] = 0.0;
  if (!probe(st.rhs, p, v0) || !(v0 > 1.0) || !std::isfinite(v0)) return false;
  eps = 1.0 / (v0 * v0);
  p.scalars[q] = 2.0 * n;
  return probe(st.rhs, p, v1) && near(v1, 1.0 / sqrt(2.0 + eps)) && eps > 1e-14 && eps < 1.0;
}
// y[r, i] = t * gamma[i] + beta[i] with t the normalised element; gamma / beta optional.  `set_t` puts the probe
// values that make t = 3 (and a second time t = -0.5).
template <typename F>
static bool probe_affine_store(const Item &it, const BpNode &st, Probe &p, Route &r, F set_t) {
  if (st.t != BpNode::EXPR || st.writes.size() != 1 || !is_global_aref(it, st.writes[0], r.out) || r.out == r.a) return false;
  r.out_idx = st.writes[0].v[2];
  std::vector<int> arrs;
  global_arefs(it, st.rhs, arrs);
  std::vector<int> extra;
  for (int a : arrs)
    if (a != r.a) extra.push_back(a);
  if (extra.size() > 2 || std::find(extra.begin(), extra.end(), r.out) != extra.end()) return false;
  auto value = [&](double t, double g, double b, int gpos, int bpos, double &out) {
    p.arrays.clear();
    p.index.clear();
    set_t(t);
    if (gpos >= 0) p.arrays[gpos] = g;
    if (bpos >= 0) p.arrays[bpos] = b;
    return probe(st.rhs, p, out);
  };
  auto fits = [&](int gpos, int bpos) {
    double v;
    const double g = gpos >= 0 ? 1.5 : 1.0, b = bpos >= 0 ? 0.25 : 0.0;
    if (!value(3.0, g, b, gpos, bpos, v) || !near(v, 3.0 * g + b)) return false;
    const double g2 = gpos >= 0 ? -0.75 : 1.0, b2 = bpos >= 0 ? 2.0 : 0.0;
    if (!value(-0.5, g2, b2, gpos, bpos, v) || !near(v, -0.5 * g2 + b2)) return false;
    r.b = gpos, r.bias = bpos;
    if (gpos >= 0) r.b_idx = p.index[gpos];
    if (bpos >= 0) r.bias_idx = p.index[bpos];
    if (p.index.count(r.a) && !sx_equal(p.index[r.a], r.a_idx)) return false;  // a shifted / strided view of x: not this norm
    return true;
  };
  if (extra.empty()) return fits(-1, -1);
  if (extra.size() == 1) return fits(extra[0], -1) || fits(-1, extra[0]);
  return fits(extra[0], extra[1]) || fits(extra[1], extra[0]);
}
static bool rownorm_loops(const std::vector<BpNode> &b, const int *fors, int nfors, Route &r) {
  const Sx *rows = upper_bound(b[0]);
  if (!rows || !is_zero(b[0].upfrom)) return false;
  r.idx[0] = b[0].idx;
  r.bound[0] = *rows;
  for (int k = 0; k < nfors; k++) {
    const BpNode &f = b[fors[k]];
    const Sx *n = upper_bound(f);
    if (!n || !is_zero(f.upfrom) || (k && (f.idx != r.idx[1] || !sx_equal(*n, r.bound[1])))) return false;
    if (!k) r.idx[1] = f.idx, r.bound[1] = *n;
  }
  return true;
}
// for r: { s = 0; for i: s += x; u = s / n; q = 0; for i: q += (x - u)^2; rr = 1 / sqrt(q / n + eps);
//          for i: y = (x - u) * rr [* gamma[i]] [+ beta[i]] }
static bool match_layernorm(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  if (b.size() != 15) return false;
  const BpNode::T want[15] = {BpNode::FOR, BpNode::EXPR, BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR, BpNode::EXPR,
                              BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR, BpNode::FOR, BpNode::EXPR,
                              BpNode::ENDFOR, BpNode::ENDFOR};
  for (int k = 0; k < 15; k++)
    if (b[k].t != want[k]) return false;
  const int fors[3] = {2, 7, 11};
  if (!rownorm_loops(b, fors, 3, r)) return false;
  if (!b[1].declare || !is_zero(b[1].rhs) || !is_scalar_ref(b[1].writes[0])) return false;
  const std::string s = ref_name(b[1].writes[0]);
  Sx term;
  if (!reduction_term(b[3], s, "add", term) || !is_global_aref(it, term, r.a)) return false;
  r.a_idx = term.v[2];
  Probe p;
  p.it = &it;
  double n, v;
  if (!probe_row_length(r.bound[1], p, n)) return false;
  // the mean
  if (!b[5].declare || b[5].writes.size() != 1 || !is_scalar_ref(b[5].writes[0])) return false;
  const std::string u = ref_name(b[5].writes[0]);
  p.scalars[s] = 3.5 * n;
  if (!probe(b[5].rhs, p, v) || !near(v, 3.5)) return false;
  p.scalars[s] = -n;
  if (!probe(b[5].rhs, p, v) || !near(v, -1.0)) return false;
  // the sum of squared deviations
  if (!b[6].declare || !is_zero(b[6].rhs) || !is_scalar_ref(b[6].writes[0])) return false;
  const std::string q = ref_name(b[6].writes[0]);
  if (!reduction_term(b[8], q, "add", term)) return false;
  const double xs[2] = {3.0, 0.5}, us[2] = {1.0, 2.0};
  for (int k = 0; k < 2; k++) {
    p.arrays.clear();
    p.index.clear();
    p.arrays[r.a] = xs[k];
    p.scalars[u] = us[k];
    if (!probe(term, p, v) || !near(v, (xs[k] - us[k]) * (xs[k] - us[k])) || !sx_equal(p.index[r.a], r.a_idx)) return false;
  }
  if (!probe_rstd(b[10], q, p, n, r.eps)) return false;
  const std::string rr = ref_name(b[10].writes[0]);
  auto set_t = [&](double t) {  // (x - u) * rr = t
    p.arrays[r.a] = 2.0 * t + 1.0;
    p.scalars[u] = 1.0;
    p.scalars[rr] = 0.5;
  };
  if (!probe_affine_store(it, b[12], p, r, set_t)) return false;
  r.kind = R_LAYERNORM;
  return true;
}
// for r: { q = 0; for i: q += x * x; rr = 1 / sqrt(q / n + eps); for i: y = x * rr [* w[i]] }
static bool match_rmsnorm(const Item &it, Route &r) {
  const std::vector<BpNode> &b = it.body;
  if (b.size() != 10) return false;
  const BpNode::T want[10] = {BpNode::FOR, BpNode::EXPR, BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::EXPR,
                              BpNode::FOR, BpNode::EXPR, BpNode::ENDFOR, BpNode::ENDFOR};
  for (int k = 0; k < 10; k++)
    if (b[k].t != want[k]) return false;
  const int fors[2] = {2, 6};
  if (!rownorm_loops(b, fors, 2, r)) return false;
  if (!b[1].declare || !is_zero(b[1].rhs) || !is_scalar_ref(b[1].writes[0])) return false;
  const std::string q = ref_name(b[1].writes[0]);
  Sx term;
  if (!reduction_term(b[3], q, "add", term)) return false;
  std::vector<int> arrs;
  global_arefs(it, term, arrs);
  if (arrs.size() != 1) return false;
  r.a = arrs[0];
  Probe p;
  p.it = &it;
  double n, v;
  if (!probe_row_length(r.bound[1], p, n)) return false;
  const double xs[2] = {3.0, -2.0};
  for (int k = 0; k < 2; k++) {
    p.arrays.clear();
    p.index.clear();
    p.arrays[r.a] = xs[k];
    if (!probe(term, p, v) || !near(v, xs[k] * xs[k])) return false;
  }
  r.a_idx = p.index[r.a];
  if (!probe_rstd(b[5], q, p, n, r.eps)) return false;
  const std::string rr = ref_name(b[5].writes[0]);
  auto set_t = [&](double t) {  // x * rr = t
    p.arrays[r.a] = 2.0 * t;
    p.scalars[rr] = 0.5;
  };
  if (!probe_affine_store(it, b[7], p, r, set_t) || r.bias >= 0) return false;
  r.kind = R_RMSNORM;
  return true;
}

// ------------------------------------------------------------------ rendering a kernel
static const char *kHeader =
    "\n#define _infinity __builtin_inff()\n"
    "#define _negative_infinity (-__builtin_inff())\n"
    "#define _nan __builtin_nanf(\"\")\n"
    "#define ct_max(a, b) ((a) > (b) ? (a) : (b))\n"
    "#define ct_min(a, b) ((a) < (b) ? (a) : (b))\n"
    "// reductions over the 64 lanes of a wavefront (every lane gets the result)\n"
    "#define CT_WAVE_REDUCE(name, T, OP)                                        \\\n"
    "  static __device__ __forceinline__ T name(T v) {                          \\\n"
    "    for (int o = 32; o > 0; o >>= 1) { T w = __shfl_xor(v, o, 64); v = OP; } \\\n"
    "    return v;                                                              \\\n"
    "  }\n"
    "CT_WAVE_REDUCE(ct_wave_add_f, float, v + w)\n"
    "CT_WAVE_REDUCE(ct_wave_max_f, float, ct_max(v, w))\n"
    "CT_WAVE_REDUCE(ct_wave_min_f, float, ct_min(v, w))\n"
    "CT_WAVE_REDUCE(ct_wave_mul_f, float, v * w)\n";

struct KernelRenderer {
  const Item &it;
  Rend R;
  std::map<std::string, bool> locals;
  explicit KernelRenderer(const Item &item) : it(item) {
    for (const BpNode &n : it.body)
      if (n.t == BpNode::EXPR && n.declare)
        for (const Sx &w : n.writes) locals[ref_name(w)] = true;
  }

  // an index made of loop indices, shape arguments and constants only: no temporary of the body (it may be set
  // after the place a hoisted read would go) and no element read inside it
  bool plain_index(const Sx &e) const {
    if (e.kind == Sx::SYM) return !locals.count(e.s);
    if (e.kind != Sx::LIST) return true;
    if (e.call("aref")) return false;
    for (size_t k = (e.call("cast") || e.call("const")) ? 2 : 1; k < e.n(); k++)
      if (!plain_index(e.v[k])) return false;
    return true;
  }

  // how many leading FOR nodes of the body (a perfect nest) are data-parallel
  int parallel_prefix() {
    const std::vector<BpNode> &b = it.body;
    int depth = 0;
    while (depth < (int)b.size() && b[depth].t == BpNode::FOR) {
      const BpNode &f = b[depth];
      const int j = match_end(b, depth);
      if (j != (int)b.size() - 1 - depth) break;
      bool ok = true;
      if (!f.global_scope) {
        for (int q = depth + 1; q < j && ok; q++) {
          const BpNode &n = b[q];
          if (n.t != BpNode::EXPR) continue;
          for (const Sx &w : n.writes) {
            const bool local = n.declare || is_scalar_ref(w) || locals.count(ref_name(w));
            if (!local && !uses(w, f.idx)) ok = false;
          }
        }
        if (!(is_zero(f.upfrom) && upper_bound(f))) ok = false;
      } else if (!upper_bound(f) || !is_zero(f.upfrom)) {
        ok = false;
      }
      if (!ok) break;
      depth++;
    }
    return depth;
  }

  // Row-reduction pattern inside the parallel prefix: {position of an ENDFOR: scalars to combine across lanes}.
  // found == false: the row stays in one thread.
  bool wave_reductions(int lo, int hi, std::map<int, std::vector<std::pair<std::string, std::string>>> &out) {
    const std::vector<BpNode> &b = it.body;
    int depth = 0;
    std::map<std::string, std::pair<bool, double>> init;  // scalar -> (is a constant, its value)
    std::vector<std::pair<std::string, std::string>> loop_red;
    std::vector<std::string> loop_reduced;  // targets of reductions in the loop being walked
    bool pending_bad = false;
    for (int pos = lo; pos < hi; pos++) {
      const BpNode &n = b[pos];
      if (n.t == BpNode::FOR) {
        if (++depth > 1 || n.global_scope || !is_one(n.by)) return false;
        loop_red.clear();
        loop_reduced.clear();
        pending_bad = false;
      } else if (n.t == BpNode::ENDFOR) {
        depth--;
        if (pending_bad) return false;
        if (!loop_red.empty()) out[pos] = loop_red;
        loop_red.clear();
      } else if (n.t == BpNode::IF || n.t == BpNode::ENDIF) {
        return false;
      } else {
        if (n.writes.size() != 1) return false;
        const Sx &w = n.writes[0];
        const bool scalar = is_scalar_ref(w);
        const std::string name = ref_name(w);
        if (depth == 0) {
          if (scalar) {
            double v;
            const bool c = const_value(n.rhs, v);
            init[name] = {c, c ? v : 0.0};
          }
          continue;
        }
        if (!n.reduction) {
          if (scalar) return false;  // a loop-carried scalar that is not a reduction cannot be split over lanes
          // an array store that reads a scalar reduced in this same loop (a running sum) would see a lane's
          // partial: such a row stays in one thread
          for (const std::string &t : loop_reduced)
            if (uses(n.rhs, t)) return false;
          // ... also when the reduction comes later in the loop body
          continue;
        }
        if (n.dtype != "float32") return false;  // the lane butterflies are fp32
        static const std::map<std::string, std::pair<std::string, double>> ident = {
            {"add", {"add", 0.0}}, {"max", {"max", -INFINITY}}, {"min", {"min", INFINITY}}, {"mul", {"mul", 1.0}}};
        const Sx &e = n.rhs;
        if (!scalar || !e.is_list() || e.n() != 3 || e.v[0].kind != Sx::SYM || !ident.count(e.v[0].s)) return false;
        const auto &id = ident.at(e.v[0].s);
        const bool s1 = is_ref_to(e.v[1], name), s2 = is_ref_to(e.v[2], name);
        if (s1 == s2 || uses(e.v[s1 ? 2 : 1], name)) return false;
        // lane partials combine when each starts at the identity; max / min are idempotent, so there any start
        // value that all lanes share (a scalar set before the loop) will do
        auto in = init.find(name);
        const bool at_identity = in != init.end() && in->second.first && in->second.second == id.second;
        if (!at_identity && !((id.first == "max" || id.first == "min") && in != init.end())) return false;
        loop_red.push_back({name, id.first});
        loop_reduced.push_back(name);
        // array stores earlier in this loop that read the scalar
        for (int q = pos - 1; q >= lo && b[q].t != BpNode::FOR; q--)
          if (b[q].t == BpNode::EXPR && !b[q].reduction && uses(b[q].rhs, name)) pending_bad = true;
      }
    }
    return !out.empty();
  }

  bool render(Program &pg, std::string &err) {
    const std::vector<BpNode> &b = it.body;
    std::string o;
    std::string params;
    for (const Global &g : it.globals) {
      const std::string &ct = cdtypes().at(g.dtype);
      if (!params.empty()) params += ", ";
      if (g.pointer) params += std::string(g.type == "input" ? "const " : "") + ct + "*" + (g.type == "input" ? " __restrict__ " : " ") + g.id;
      else params += "const " + ct + " " + g.id;
    }
    for (const BpNode &n : b)
      if (n.t == BpNode::EXPR && n.grid_rank >= 0) {
        if (!pg.explicit_grid)
          for (int q = 0; q < 3; q++) pg.grid_global[q] = pg.grid_local[q] = sx_int(1);
        pg.explicit_grid = true;
        pg.grid_global[n.grid_rank] = n.grid_global;
        pg.grid_local[n.grid_rank] = n.grid_local;
      }
    o += std::string("extern \"C\" __global__ void __launch_bounds__(") + (pg.explicit_grid ? "1024" : "256") + ") " + it.name + "(" + params + ") {\n";
    // an item that brings its own grid keeps its loops as they are: the scheduler has distributed it already
    const int npar = pg.explicit_grid ? 0 : parallel_prefix();
    std::map<int, std::vector<std::pair<std::string, std::string>>> wave_red;
    const int lo = npar, hi = (int)b.size() - npar;
    const bool wave = npar > 0 && wave_reductions(lo, hi, wave_red);
    // Element-wise items (no loop inside the parallel prefix, no wavefront reduction): a thread takes FOUR elements,
    // 256 apart, so that each of its four loads and stores is a contiguous 1 KB per wavefront pair and the four are
    // in flight together.  One element per thread left the 50 M-element GELU at 123 (static) / 149 us (run-time
    // shape, where every thread also paid two 64-bit divisions) against 75 us of the hand-written kernel.
    bool flat4 = npar > 0 && !wave && !pg.explicit_grid;
    for (int pos = lo; pos < hi && flat4; pos++)
      if (b[pos].t == BpNode::FOR) flat4 = false;
    pg.rows_per_block = wave ? 4 : flat4 ? 1024 : 256;
    pg.parallel = npar > 0;
    int indent = 2;
    auto pad = [&]() { return std::string((size_t)indent, ' '); };
    // _t -> the loop indices, innermost fastest; the outermost needs no remainder (_t < _total).  wide: 0 = 32-bit
    // arithmetic (the caller has tested _total <= 0x7fffffff), 1 = 64-bit, -1 = that test here, around both
    auto decompose = [&](int wide) {
      if (npar == 1) {
        o += pad() + "const int " + b[0].idx + " = (int)_t;\n";
        return;
      }
      std::string decl = pad() + "int ";
      for (int q = 0; q < npar; q++) decl += std::string(q ? ", " : "") + b[q].idx;
      o += decl + ";\n";
      for (int w = 0; w < 2; w++) {
        if (wide >= 0 && wide != w) continue;
        const std::string ty = w ? "long long" : "unsigned";
        o += pad() + (wide >= 0 ? "{" : w ? "} else {" : "if (_total <= 0x7fffffffLL) {") + " " + ty + " _u = (" + ty + ")_t;";
        for (int q = npar - 1; q >= 1; q--) {
          const std::string bs = "(" + ty + ")(" + R.expr(*upper_bound(b[q]), "int64") + ")";
          double cv;
          if (!w && !const_value(*upper_bound(b[q]), cv))
            // a bound known at launch only, 32 bits: quotient by the rounded-down reciprocal floor((2^32 - 1) / n) --
            // one division per thread instead of one per element; it comes out at most one too small for _u < 2^31
            o += " { const unsigned _n = " + bs + "; unsigned _q = __umulhi(_u, 0xffffffffu / _n), _r = _u - _q * _n; if (_r >= _n) { _r -= _n; _q++; } " +
                 b[q].idx + " = (int)_r; _u = _q; }";
          else
            o += " " + b[q].idx + " = (int)(_u % " + bs + "); _u /= " + bs + ";";
        }
        o += " " + b[0].idx + " = (int)_u;" + (wide >= 0 ? " }" : "") + "\n";
      }
      if (wide < 0) o += pad() + "}\n";
    };
    if (npar) {
      std::string total;
      for (int q = 0; q < npar; q++) {
        const Sx *ub = upper_bound(b[q]);
        pg.grid_bounds.push_back(*ub);
        total += std::string(q ? "*" : "") + "(long long)(" + R.expr(*ub, "int64") + ")";
      }
      o += pad() + "const long long _total = " + total + ";\n";
      if (wave) {
        o += pad() + "long long _t = ((long long)blockIdx.x * 256 + threadIdx.x) >> 6;  // one wavefront per row\n";
        o += pad() + "const int _lane = threadIdx.x & 63;\n";
      } else if (!flat4) {
        o += pad() + "long long _t = (long long)blockIdx.x * 256 + threadIdx.x;\n";
      }
      if (!flat4) {
        o += pad() + "if (_t >= _total) return;\n";
        decompose(-1);
      }
    }
    // row loops of the wavefront path whose length is only known at run time (from 0, step 1)
    std::map<int, bool> dyn_rows;
    std::string dyn_cond, dyn_nonempty;
    bool dyn_ok = true;
    if (wave) {
      for (int pos = lo; pos < hi; pos++) {
        const BpNode &n = b[pos];
        if (n.t != BpNode::FOR) continue;
        double v;
        const Sx *ub = upper_bound(n);
        if (!ub || const_value(*ub, v) || !is_zero(n.upfrom)) continue;
        bool inner = false;  // only loops directly inside the row (depth 0 of the body)
        int d = 0;
        for (int q = lo; q < pos; q++) d += b[q].t == BpNode::FOR ? 1 : b[q].t == BpNode::ENDFOR ? -1 : 0;
        inner = d == 0;
        if (!inner) continue;
        dyn_rows[pos] = true;
        const std::string c = "(" + R.expr(*ub, "int64") + ") <= 2048", c0 = "(" + R.expr(*ub, "int64") + ") > 0";
        if (dyn_cond.find(c) == std::string::npos) dyn_cond += std::string(dyn_cond.empty() ? "" : " && ") + c;
        if (dyn_nonempty.find(c0) == std::string::npos) dyn_nonempty += std::string(dyn_nonempty.empty() ? "" : " && ") + c0;
      }
    }
    // bounded: row loops of dynamic length are emitted as 32 counted, unrolled, guarded passes (the caller has
    // checked at run time that the row has at most 64 * 32 elements), so that, as for a static row, the loops
    // over the same row can share their loads and the row is read once
    // The loops over one dynamic row read the same elements.  The compiler merges equal loads only over a short
    // distance, and a load that follows a store to an unqualified pointer is repeated, one round trip per
    // element; so the elements that the row's loops read from the kernel's INPUT arrays (never written here) are
    // loaded once, into registers, by a pass of their own in front of the first loop, and the loops read those.
    // Only loops with the first one's index name and bound take part (their pass counters mean the same element).
    // siblings: the row loops that take part; head / close: what opens and closes one pass over the row (the loops
    // and any guard, as the row's own loops are opened); dims / slot: the shape of a register array that holds one
    // value per element of the thread, and the element's place in it
    auto hold_loops = [&](const std::vector<int> &siblings, const std::string &head, const std::string &close, const std::string &idx,
                          const std::string &dims, const std::string &slot, int per_thread, std::string &out, const std::string &ind) {
      std::vector<std::pair<std::string, std::string>> refs;  // rendered reference, element type
      std::function<void(const Sx &)> walk = [&](const Sx &e) {
        if (e.call("where")) return;  // an arm of a `where` may be what keeps an index inside its array: not hoisted
        if (e.call("aref") && e.n() >= 3 && !e.v[2].is_sym("nil")) {
          const int g = arg_pos(it, e.v[1].s);
          if (g >= 0 && it.globals[g].pointer && it.globals[g].type == "input" && uses(e.v[2], idx) && plain_index(e.v[2])) {
            const std::string ref = R.aref(e);
            bool seen = false;
            for (const auto &r : refs) seen = seen || r.first == ref;
            if (!seen) refs.push_back({ref, cdtypes().at(it.globals[g].dtype)});
          }
          return;
        }
        if (e.kind == Sx::LIST)
          for (const Sx &c : e.v) walk(c);
      };
      for (int f : siblings)
        for (int q = f + 1; q < hi && b[q].t != BpNode::ENDFOR; q++) {
          if (b[q].t != BpNode::EXPR) return;  // something else than statements in a row loop: hold nothing
          walk(b[q].rhs);
        }
      if (refs.empty() || refs.size() > 4 || (int)refs.size() * per_thread > 96) return;
      for (size_t k = 0; k < refs.size(); k++) out += ind + refs[k].second + " _h" + std::to_string(k) + dims + ";\n";
      out += ind + "#pragma unroll\n";
      out += ind + head;
      for (size_t k = 0; k < refs.size(); k++) out += " _h" + std::to_string(k) + slot + " = " + refs[k].first + ";";
      out += " " + close + "\n";
      for (size_t k = 0; k < refs.size(); k++) R.held[refs[k].first] = "_h" + std::to_string(k) + slot;
    };
    // dynamic rows: the loops with the first one's index name; another range under the same name: hold nothing
    auto hold_row = [&](int first, const std::string &head, const std::string &idx, const std::string &ub_s, int passes, std::string &out,
                        const std::string &ind) {
      std::vector<int> siblings;
      for (const auto &kv : dyn_rows) {
        const BpNode &f = b[kv.first];
        if (f.idx != idx) continue;
        if (R.expr(*upper_bound(f), "int64") != ub_s) return;
        siblings.push_back(kv.first);
      }
      (void)first;
      hold_loops(siblings, head, "}", idx, "[" + std::to_string(passes) + "]", "[" + idx + "_i]", passes, out, ind);
    };
    // static rows: the loops directly inside the row with this loop's index name, which must all have its range;
    // at least two of them (a row that is walked once gains nothing), and this one the first
    auto static_siblings = [&](int pos, long long l, long long h) {
      std::vector<int> sib;
      int d = 0;
      for (int q = lo; q < hi; q++) {
        if (b[q].t == BpNode::FOR) {
          if (d == 0 && b[q].idx == b[pos].idx) {
            double fl, fh;
            const Sx *ub = upper_bound(b[q]);
            if (!ub || !const_value(b[q].upfrom, fl) || !const_value(*ub, fh) || (long long)fl != l || (long long)fh != h) return std::vector<int>();
            sib.push_back(q);
          }
          d++;
        } else if (b[q].t == BpNode::ENDFOR) {
          d--;
        }
      }
      if (sib.size() < 2 || sib[0] != pos) sib.clear();
      return sib;
    };
    const std::vector<std::pair<std::string, std::string>> *held_flat = nullptr;   // element-wise items: reads held per element
    const std::vector<std::pair<std::string, std::string>> *flat_named = nullptr;  // ... and elements addressed by _t
    auto emit_body = [&](int bounded) {  // 0: lane-strided loops; N: dynamic rows as N counted passes
    R.held.clear();
    if (flat_named)
      for (const auto &fr : *flat_named) R.held[fr.first] = fr.second;
    if (held_flat)
      for (size_t k = 0; k < held_flat->size(); k++) R.held[(*held_flat)[k].first] = "_h" + std::to_string(k) + "[_e]";
    int depth = 0;
    std::string guard;  // inside a counted pass of a dynamic row: the name of its "this element exists" flag
    std::vector<std::string> closers;
    for (int pos = lo; pos < hi; pos++) {
      const BpNode &n = b[pos];
      if (n.t == BpNode::FOR) {
        bool done = false;
        if (wave) {  // the lanes of the row's wavefront stride this axis together
          double flo, fhi;
          const Sx *ub = upper_bound(n);
          if (ub && const_value(n.upfrom, flo) && const_value(*ub, fhi) && flo == floor(flo) && fhi == floor(fhi)) {
            const long long l = (long long)flo, h = (long long)fhi, per = (h - l + 63) / 64, quads = (h - l) / 4;
            if ((h - l) % 4 == 0 && quads >= 64 && (quads + 63) / 64 <= 8) {
              // a row of whole quads, at least one per lane: a lane owns 4 CONSECUTIVE elements per pass, so its four
              // loads (and stores) of a stride-1 operand are one 128-bit access after the compiler has merged them
              const long long per4 = (quads + 63) / 64;
              const bool ragged = quads % 64 != 0;
              const std::string h1 = "for (int " + n.idx + "_i=0; " + n.idx + "_i<" + std::to_string(per4) + "; " + n.idx + "_i++) {" +
                                     (ragged ? " const bool " + n.idx + "_q=_lane+64*" + n.idx + "_i<" + std::to_string(quads) + ";" : "");
              const std::string h2 = "for (int " + n.idx + "_k=0; " + n.idx + "_k<4; " + n.idx + "_k++) { const int " + n.idx + "=" + std::to_string(l) +
                                     "+4*(_lane+64*" + n.idx + "_i)+" + n.idx + "_k;" + (ragged ? " if (" + n.idx + "_q) {" : "");
              if (depth == 0) {
                const std::vector<int> sib = static_siblings(pos, l, h);
                if (!sib.empty())
                  hold_loops(sib, h1 + "\n" + pad() + "#pragma unroll\n" + pad() + h2, ragged ? "}}}" : "}}", n.idx, "[" + std::to_string(per4) + "][4]",
                             "[" + n.idx + "_i][" + n.idx + "_k]", (int)per4 * 4, o, pad());
              }
              o += pad() + "#pragma unroll\n";
              o += pad() + h1 + "\n";
              o += pad() + "#pragma unroll\n";
              o += pad() + h2 + "\n";
              closers.push_back(ragged ? "}}}" : "}}");
              done = true;
            } else if (per > 0 && per <= 32) {
              // a static row of at most 32 elements per lane: a counted loop, unrolled, so that the loops over the
              // same row share their loads (inputs are __restrict__) and the row is read once
              const bool ragged = (h - l) % 64 != 0;
              const std::string h1 = "for (int " + n.idx + "_i=0; " + n.idx + "_i<" + std::to_string(per) + "; " + n.idx + "_i++) { const int " + n.idx + "=" +
                                     std::to_string(l) + "+_lane+64*" + n.idx + "_i;" + (ragged ? " if (" + n.idx + "<" + std::to_string(h) + ") {" : "");
              if (depth == 0) {
                const std::vector<int> sib = static_siblings(pos, l, h);
                if (!sib.empty())
                  hold_loops(sib, h1, ragged ? "}}" : "}", n.idx, "[" + std::to_string(per) + "]", "[" + n.idx + "_i]", (int)per, o, pad());
              }
              o += pad() + "#pragma unroll\n";
              o += pad() + h1 + "\n";
              closers.push_back(ragged ? "}}" : "}");
              done = true;
            }
          }
          if (!done && bounded && dyn_rows.count(pos)) {
            // every pass reads unconditionally (the index is clamped to the row's last element) and only its
            // effects are guarded: the loads of the loops over one row are then the same expressions and are shared
            const std::string ub_s = R.expr(*upper_bound(n), "int64");
            const std::string head = "for (int " + n.idx + "_i=0; " + n.idx + "_i<" + std::to_string(bounded) + "; " + n.idx + "_i++) { const bool " + n.idx +
                                     "_ok=_lane+64*" + n.idx + "_i<(" + ub_s + "); const int " + n.idx + "=" + n.idx + "_ok ? _lane+64*" + n.idx + "_i : (int)(" + ub_s + ")-1;";
            if (pos == dyn_rows.begin()->first) hold_row(pos, head, n.idx, ub_s, bounded, o, pad());
            o += pad() + "#pragma unroll\n";
            o += pad() + head + "\n";
            closers.push_back("}");
            guard = n.idx + "_ok";
            done = true;
          }
          if (!done) {
            o += pad() + "for (int " + n.idx + "=(" + R.expr(n.upfrom, "int64") + ")+_lane; " + R.expr(n.below, "int64") + "; " + n.idx + "+=64) {\n";
            closers.push_back("}");
          }
        } else {
          o += pad() + "for (int " + n.idx + "=" + R.expr(n.upfrom, "int64") + "; " + R.expr(n.below, "int64") + "; " + n.idx + "+=" +
               R.expr(n.by, "int64") + ") {\n";
          closers.push_back("}");
        }
        indent += 2;
        depth++;
      } else if (n.t == BpNode::ENDFOR) {
        indent -= 2;
        depth--;
        if (depth == 0) guard.clear();
        o += pad() + closers.back() + "\n";
        closers.pop_back();
        if (wave && wave_red.count(pos))
          for (const auto &vr : wave_red[pos]) o += pad() + vr.first + " = ct_wave_" + vr.second + "_f(" + vr.first + ");\n";
      } else if (n.t == BpNode::IF) {
        o += pad() + "if (" + R.expr(n.cond, "int64") + ") {\n";
        indent += 2;
      } else if (n.t == BpNode::ENDIF) {
        indent -= 2;
        o += pad() + "}\n";
      } else {
        std::string lhs;
        for (size_t k = 0; k < n.writes.size(); k++) lhs += std::string(k ? ", " : "") + (n.writes[k].kind == Sx::SYM ? n.writes[k].s : R.aref(n.writes[k]));
        std::string stmt = (n.declare ? cdtypes().at(n.dtype) + " " : "") + lhs + " = " + R.expr(n.rhs, n.dtype) + ";";
        bool global_write = false;
        for (const Sx &w : n.writes)
          if (!locals.count(ref_name(w))) global_write = true;
        if (wave && depth == 0 && !n.declare && global_write) stmt = "if (_lane == 0) { " + stmt + " }";  // every lane holds the value; one stores it
        if (depth == 1 && !guard.empty()) {
          // the value is computed outside the guard, on the clamped index the other loops use, so that it is shared
          if (global_write && n.writes.size() == 1 && !uses(n.rhs, ref_name(n.writes[0]))) {
            // a pass beyond the row repeats the store of the row's last element, with the same value: no guard at
            // all (a guarded store takes the loads it depends on into its branch, one round trip each)
          } else if (global_write && n.writes.size() == 1)
            stmt = "{ const " + cdtypes().at(n.dtype) + " _w = " + R.expr(n.rhs, n.dtype) + "; if (" + guard + ") { " + lhs + " = _w; } }";
          else if (global_write) stmt = "if (" + guard + ") { " + stmt + " }";
          else if (!n.declare && n.writes.size() == 1)
            // (as a statement of its own: inside the conditional operator the reads would be conditional as well, and a
            // conditional load waits for its answer before the next one is asked for)
            stmt = "{ const " + cdtypes().at(n.dtype) + " _w = " + R.expr(n.rhs, n.dtype) + "; " + lhs + " = " + guard + " ? _w : " + lhs + "; }";
        }
        o += pad() + stmt + "\n";
      }
    }
    R.held.clear();
    };
    if (dyn_rows.size() < 2) dyn_rows.clear();  // a row that is walked once gains nothing from being held
    for (const auto &kv : dyn_rows) {            // row loops with nothing but statements inside, and a non-empty row
      for (int q = kv.first + 1; q < hi && b[q].t != BpNode::ENDFOR; q++)
        if (b[q].t != BpNode::EXPR || b[q].declare) dyn_ok = false;
    }
    if (!dyn_rows.empty() && dyn_ok) {
      // copies of the body for rows of up to 256 ... 2048 elements (4 ... 32 passes: a pass beyond the row still
      // computes on the clamped element), then the loops
      const int passes[6] = {4, 8, 12, 16, 24, 32};
      for (int k = 0; k < 6; k++) {
        std::string c = dyn_cond;
        for (size_t at = c.find("<= 2048"); at != std::string::npos; at = c.find("<= 2048", at + 1)) c.replace(at, 7, "<= " + std::to_string(64 * passes[k]));
        o += pad() + (k ? "} else if (" : "if (") + dyn_nonempty + " && " + c + ") {\n";
        indent += 2;
        emit_body(passes[k]);
        indent -= 2;
      }
      o += pad() + "} else {\n";
      indent += 2;
      emit_body(0);
      indent -= 2;
      o += pad() + "}\n";
    } else if (flat4) {
      // whole blocks of 1024 elements run without a test; the last, partial one tests every element.  Each in a
      // 32-bit and a 64-bit copy (several indices to take apart): a test inside the element loop would keep the four
      // elements' loads from being issued together
      o += pad() + "const long long _b0 = (long long)blockIdx.x * 1024 + threadIdx.x;\n";
      const int nwide = npar > 1 ? 2 : 1;
      // the elements that the statements read from INPUT arrays are loaded by a loop of their own in front of
      // the statements' loop, so that the four elements' loads are under way together whatever the statements
      // store in between (not under a condition: an IF node or the arm of a `where` may be what keeps an index
      // inside its array)
      // An element whose index IS the row-major position over the parallel loops (sum of index x the bounds inside
      // it) is addressed by _t itself: no multiplications, and the accesses are visibly consecutive.  Recognised by
      // value: the index expression is evaluated at a few points (shape arguments, bounds and indices set to
      // unrelated numbers) against that sum.
      auto flat_index = [&](const Sx &idx) {
        static const double primes[8] = {101, 211, 307, 401, 503, 601, 701, 809};
        for (int trial = 0; trial < 4; trial++) {
          Probe pr;
          pr.it = &it;
          int k = 0;
          for (const Global &g : it.globals)
            if (!g.pointer) pr.scalars[g.id] = primes[(k++ + 3 * trial) % 8] + trial;
          double flat = 0.0, inner = 1.0;
          for (int q = npar - 1; q >= 0; q--) {
            double bq;
            if (!probe(*upper_bound(b[q]), pr, bq) || bq < 1.0) return false;
            const double gq = fmod(primes[(q + 5 * trial + 1) % 8] * 13.0 + q, bq);
            pr.scalars[b[q].idx] = gq;
            flat += gq * inner;
            inner *= bq;
          }
          double v;
          if (!probe(idx, pr, v) || !near(v, flat)) return false;
        }
        return true;
      };
      std::vector<std::pair<std::string, std::string>> flat_refs;  // rendered reference -> the same element by _t
      {
        std::function<void(const Sx &)> walk = [&](const Sx &e) {
          if (e.call("aref") && e.n() >= 3 && !e.v[2].is_sym("nil")) {
            const int g = arg_pos(it, e.v[1].s);
            if (g >= 0 && it.globals[g].pointer && flat_index(e.v[2])) {
              const std::string ref = R.aref(e);
              bool seen = false;
              for (const auto &r : flat_refs) seen = seen || r.first == ref;
              if (!seen) flat_refs.push_back({ref, e.v[1].s + "[_t]"});
            }
            return;
          }
          if (e.kind == Sx::LIST)
            for (const Sx &c : e.v) walk(c);
        };
        for (int pos = lo; pos < hi; pos++)
          if (b[pos].t == BpNode::EXPR) {
            walk(b[pos].rhs);
            for (const Sx &w : b[pos].writes) walk(w);
          }
      }
      std::vector<std::pair<std::string, std::string>> refs;  // rendered reference, element type
      {
        bool plain = true;
        for (int pos = lo; pos < hi; pos++) plain = plain && b[pos].t == BpNode::EXPR;
        std::function<void(const Sx &)> walk = [&](const Sx &e) {
          if (e.call("where")) return;
          if (e.call("aref") && e.n() >= 3 && !e.v[2].is_sym("nil")) {
            const int g = arg_pos(it, e.v[1].s);
            if (g >= 0 && it.globals[g].pointer && it.globals[g].type == "input" && plain_index(e.v[2])) {
              const std::string ref = R.aref(e);
              bool seen = false;
              for (const auto &r : refs) seen = seen || r.first == ref;
              if (!seen) refs.push_back({ref, cdtypes().at(it.globals[g].dtype)});
            }
            return;
          }
          if (e.kind == Sx::LIST)
            for (const Sx &c : e.v) walk(c);
        };
        if (plain)
          for (int pos = lo; pos < hi; pos++) walk(b[pos].rhs);
        if (refs.size() > 6) refs.clear();
      }
      for (int w = 0; w < nwide; w++) {
        if (nwide == 2) {
          o += pad() + (w ? "} else {" : "if (_total <= 0x7fffffffLL) {") + "\n";
          indent += 2;
        }
        for (int tail = 0; tail < 2; tail++) {
          o += pad() + (tail ? "} else {" : "if ((long long)blockIdx.x * 1024 + 1024 <= _total) {") + "\n";
          indent += 2;
          const std::string head = std::string("for (int _e = 0; _e < 4; _e++) { const long long _t = _b0 + 256 * _e;") + (tail ? " if (_t < _total) {" : "");
          if (!refs.empty()) {
            for (size_t k = 0; k < refs.size(); k++) o += pad() + refs[k].second + " _h" + std::to_string(k) + "[4];\n";
            o += pad() + "#pragma unroll\n";
            o += pad() + head + "\n";
            indent += 2;
            decompose(w);
            for (size_t k = 0; k < refs.size(); k++) {
              std::string from = refs[k].first;
              for (const auto &fr : flat_refs)
                if (fr.first == from) from = fr.second;
              o += pad() + "_h" + std::to_string(k) + "[_e] = " + from + ";\n";
            }
            indent -= 2;
            o += pad() + (tail ? "}}" : "}") + "\n";
          }
          o += pad() + "#pragma unroll\n";
          o += pad() + head + "\n";
          indent += 2;
          decompose(w);
          held_flat = &refs;
          flat_named = &flat_refs;
          emit_body(0);
          held_flat = flat_named = nullptr;
          indent -= 2;
          o += pad() + (tail ? "}}" : "}") + "\n";
          indent -= 2;
        }
        o += pad() + "}\n";
        if (nwide == 2) indent -= 2;
      }
      if (nwide == 2) o += pad() + "}\n";
    } else {
      dyn_rows.clear();
      emit_body(0);
    }
    o += "}\n";
    if (!R.err.empty()) return err = R.err, false;
    pg.source = o;
    return true;
  }
};

// entry points of the hand-written kernels the routes use (matmul.hip, linear.hip, rowops.hip)
int matmul_routed(float *C, const float *A, const float *B, int M, int N, int K, int act, const float *bias, const float *residual,
                  bool b_is_nk);
int launch_embedding(float *out, const float *W, const float *idx_f, const int *idx_i, int ntok, int vocab, int dim,
                     const float *W2, const int *pos, int max_pos);
int launch_embedding_rows(float *out, const float *W, long long first, long long step, int ntok, int vocab, int dim, const float *addend);

static bool launch_route(Program &pg, void **args, const std::map<std::string, long long> &env, int &rc) {
  Route &r = pg.route;
  rc = 0;
  auto ptr = [&](int pos) { return *(void **)args[pos]; };
  auto bound = [&](int q, long long &v) { return eval_int(r.bound[q], env, v) && v >= 0 && v <= 0x7fffffff; };
  auto aligned = [](const float *p) { return ((uintptr_t)p % 16) == 0; };
  if (r.kind == R_MATMUL) {
    const int nl = (int)r.lidx.size(), P = nl - 1;  // loops: batch..., i, j, then k
    const int ii = P - 2, jj = P - 1, kk = P;
    std::vector<long long> key;
    key.reserve(env.size());
    for (const auto &kv : env) key.push_back(kv.second);
    if (!pg.memo_ok || key != pg.memo_key) {
      pg.memo_ok = false;
      pg.memo_key = key;
      pg.memo_ext.assign(nl, 0);
      for (int q = 0; q < nl; q++)
        if (!eval_int(r.lbound[q], env, pg.memo_ext[q]) || pg.memo_ext[q] < 0 || pg.memo_ext[q] > 0x7fffffff) return false;
      if (!affine_n(r.out_idx, r.lidx, env, pg.memo_aff[0]) || !affine_n(r.a_idx, r.lidx, env, pg.memo_aff[1]) ||
          !affine_n(r.b_idx, r.lidx, env, pg.memo_aff[2]))
        return false;
      // the result does not move with k, A not with j, B not with i
      if (pg.memo_aff[0].c[kk] || pg.memo_aff[1].c[jj] || pg.memo_aff[2].c[ii]) return false;
      for (int q = 0; q < 2; q++)
        if (r.extra[q] >= 0 && (!affine_n(r.extra_idx[q], r.lidx, env, pg.memo_aff[3 + q]) || pg.memo_aff[3 + q].c[kk])) return false;
      pg.memo_ok = true;
    }
    const std::vector<long long> &ext = pg.memo_ext;
    const long long M = ext[P - 2], N = ext[P - 1], K = ext[P];
    long long nbatch = 1;
    for (int q = 0; q < P - 2; q++) nbatch *= ext[q];
    const AffineN &ao = pg.memo_aff[0], &aa = pg.memo_aff[1], &ab = pg.memo_aff[2];
    const AffineN *ae = pg.memo_aff + 3;
    if (M == 0 || N == 0 || nbatch == 0) return true;
    if (ao.base < 0 || aa.base < 0 || ab.base < 0) return false;
    float *C = (float *)ptr(r.out) + ao.base;
    const float *A = (const float *)ptr(r.a) + aa.base, *B = (const float *)ptr(r.b) + ab.base;
    // (1) one dense row-major product: the MFMA GEMM, or the single-row kernels for a few rows of a Linear
    bool b_nk = false;
    bool dense = nbatch == 1 && r.alpha == 1.0 && ao.c[ii] == N && ao.c[jj] == 1 && aa.c[ii] == K && aa.c[kk] == 1 && aligned(C) && aligned(A) && aligned(B);
    if (dense) {
      if (ab.c[jj] == 1 && ab.c[kk] == N) b_nk = false;       // B (K,N) row-major
      else if (ab.c[jj] == K && ab.c[kk] == 1) b_nk = true;   // W (N,K) read through a transposed view
      else dense = false;
    }
    const float *bias = nullptr, *resid = nullptr;
    for (int q = 0; q < 2 && dense; q++) {
      if (r.extra[q] < 0) continue;
      if (ae[q].base < 0) return false;
      const float *e = (const float *)ptr(r.extra[q]) + ae[q].base;
      const bool by_col = ae[q].c[ii] == 0 && ae[q].c[jj] == 1, full = ae[q].c[ii] == N && ae[q].c[jj] == 1;
      // without an activation "before" and "after" are the same thing
      const bool may_pre = !r.extra_post[q] || r.act == CTHIP_ACT_NONE, may_post = r.extra_post[q] || r.act == CTHIP_ACT_NONE;
      if (by_col && may_pre && !bias && aligned(e)) bias = e;
      else if (full && may_post && !resid && aligned(e)) resid = e;
      else dense = false;
    }
    if (dense) {
      rc = matmul_routed(C, A, B, (int)M, (int)N, (int)K, r.act, bias, resid, b_nk);
      pg.last_route = b_nk ? "cthip_linear" : "cthip_matmul";
      return true;
    }
    // (2) batched / strided / scaled: the attention items over the cache view, chunked operands
    if (P - 2 > 3) return false;
    BmmArgs g = {};
    g.C = (float *)ptr(r.out);
    g.A = (const float *)ptr(r.a);
    g.B = (const float *)ptr(r.b);
    auto fill = [&](BmmOperand &o, const AffineN &f) {
      o.base = f.base;
      for (int q = 0; q < 3; q++) o.sb[q] = q < P - 2 ? f.c[q] : 0;
      o.si = f.c[ii];
      o.sj = f.c[jj];
      o.sk = f.c[kk];
    };
    fill(g.c, ao);
    fill(g.a, aa);
    fill(g.b, ab);
    for (int q = 0; q < 3; q++) g.nb[q] = q < P - 2 ? (int)ext[q] : 1;
    g.M = (int)M, g.N = (int)N, g.K = (int)K;
    g.alpha = (float)r.alpha;
    g.act = r.act;
    for (int q = 0; q < 2; q++) {
      if (r.extra[q] < 0) continue;
      if (ae[q].base < 0) return false;
      const float *e = (const float *)ptr(r.extra[q]);
      if (r.extra_post[q]) {
        if (g.post) return false;
        g.post = e;
        fill(g.r, ae[q]);
      } else if (!g.pre0) {
        g.pre0 = e;
        fill(g.p0, ae[q]);
      } else {
        g.pre1 = e;
        fill(g.p1, ae[q]);
      }
    }
    if (K == 0 || !bmm_variant(g)) return false;
    rc = launch_bmm(g);
    pg.last_route = "cthip_bmm";
    return true;
  }
  if (r.kind == R_EMBEDDING) {
    long long T, D, V;
    if (!bound(0, T) || !bound(1, D) || !bound(2, V)) return false;
    Affine ao, aw, ai;
    if (!affine_of(r.out_idx, r.idx, 3, env, ao) || !affine_of(r.a_idx, r.idx, 3, env, aw) || !affine_of(r.b_idx, r.idx, 3, env, ai)) return false;
    if (ao.base || ao.c[0] != D || ao.c[1] != 1 || ao.c[2]) return false;  // out (T, D)
    if (aw.base || aw.c[0] || aw.c[1] != 1 || aw.c[2] != D) return false;  // W (V, D)
    Affine av;
    if (!affine_of(r.bias_idx, r.idx, 3, env, av) || av.base || av.c[0] || av.c[1] || av.c[2] != 1) return false;  // compared with v itself
    const float *addend = nullptr;
    if (r.extra[0] >= 0) {  // + other[t, d]
      Affine ae;
      if (!affine_of(r.extra_idx[0], r.idx, 3, env, ae) || ae.base || ae.c[0] != D || ae.c[1] != 1 || ae.c[2]) return false;
      addend = (const float *)ptr(r.extra[0]);
    }
    if (r.b < 0) {
      // rows first, first + step, ...: token position t selects row (first + step * t)
      if (ai.c[1] || ai.c[2]) return false;
      if (T == 0 || D == 0) return true;
      rc = launch_embedding_rows((float *)ptr(r.out), (const float *)ptr(r.a), ai.base, ai.c[0], (int)T, (int)V, (int)D, addend);
      pg.last_route = "cthip_embedding";
      return true;
    }
    if (addend) return false;
    if (ai.base || ai.c[0] != 1 || ai.c[1] || ai.c[2]) return false;       // idx (T)
    if (T == 0 || D == 0) return true;
    rc = cthip_embedding((float *)ptr(r.out), (const float *)ptr(r.a), (const float *)ptr(r.b), (int)T, (int)V, (int)D);
    pg.last_route = "cthip_embedding";
    return true;
  }
  if (r.kind == R_ARGMAX) {
    long long Rn, N;
    if (!bound(0, Rn) || !bound(1, N) || N < 1) return false;
    Affine ax, ao;
    // (a base offset = a view from some row on: the last position's logits, external/llm/layers.lisp:90)
    if (!affine_of(r.a_idx, r.idx, 2, env, ax) || ax.base < 0 || (ax.c[0] != N && Rn > 1) || ax.c[1] != 1) return false;
    const std::string oi[3] = {r.idx[0], "", ""};
    if (!affine_of(r.out_idx, oi, 1, env, ao) || ao.base || (ao.c[0] != 1 && Rn > 1)) return false;
    // kept value (N - 1) - i and result N - g - 1, whatever their spelling
    std::map<std::string, long long> e2 = env;
    for (long long i : {0ll, 1ll, N - 1}) {
      e2[r.idx[1]] = i;
      e2[r.idx[2]] = i;
      long long v;
      if (!eval_int(r.b_idx, e2, v) || v != (N - 1) - i) return false;
    }
    for (long long g : {0ll, N - 1}) {
      e2[r.bound[2].s] = g;
      long long v;
      if (!eval_int(r.bias_idx, e2, v) || v != N - g - 1) return false;
    }
    if (Rn == 0) return true;
    rc = cthip_argmax((int64_t *)ptr(r.out), (const float *)ptr(r.a) + ax.base, Rn, (int)N);
    pg.last_route = "cthip_argmax";
    return true;
  }
  if (r.kind == R_SOFTMAX) {
    long long Rn, N;
    if (!bound(0, Rn) || !bound(1, N) || N < 1) return false;
    Affine ax, ao;
    if (!affine_of(r.a_idx, r.idx, 2, env, ax) || ax.base || ax.c[0] != N || ax.c[1] != 1) return false;
    if (!affine_of(r.out_idx, r.idx, 2, env, ao) || ao.base || ao.c[0] != N || ao.c[1] != 1) return false;
    if (Rn == 0) return true;
    rc = cthip_softmax((float *)ptr(r.out), (const float *)ptr(r.a), Rn, (int)N);
    pg.last_route = "cthip_softmax";
    return true;
  }
  if (r.kind == R_LAYERNORM || r.kind == R_RMSNORM) {
    long long Rn, N;
    if (!bound(0, Rn) || !bound(1, N) || N < 1) return false;
    Affine ax, ao, ag;
    if (!affine_of(r.a_idx, r.idx, 2, env, ax) || ax.base || ax.c[0] != N || ax.c[1] != 1) return false;
    if (!affine_of(r.out_idx, r.idx, 2, env, ao) || ao.base || ao.c[0] != N || ao.c[1] != 1) return false;
    // gamma / beta are read by column, whatever the row
    if (r.b >= 0 && (!affine_of(r.b_idx, r.idx, 2, env, ag) || ag.base || ag.c[0] != 0 || ag.c[1] != 1)) return false;
    if (r.bias >= 0 && (!affine_of(r.bias_idx, r.idx, 2, env, ag) || ag.base || ag.c[0] != 0 || ag.c[1] != 1)) return false;
    if (Rn == 0) return true;
    const float *g = r.b >= 0 ? (const float *)ptr(r.b) : nullptr, *bt = r.bias >= 0 ? (const float *)ptr(r.bias) : nullptr;
    if (r.kind == R_LAYERNORM) {
      rc = cthip_layernorm((float *)ptr(r.out), (const float *)ptr(r.a), g, bt, (float)r.eps, Rn, (int)N);
      pg.last_route = "cthip_layernorm";
    } else {
      rc = cthip_rmsnorm((float *)ptr(r.out), (const float *)ptr(r.a), g, (float)r.eps, Rn, (int)N);
      pg.last_route = "cthip_rmsnorm";
    }
    return true;
  }
  return false;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

const char *cthip_render_header(void) { return kHeader; }

int cthip_program_create(void **program, const char *blueprint) {
  CTHIP_ARG(program != nullptr && blueprint != nullptr);
  Parser ps{blueprint, {}};
  Sx top;
  if (!ps.parse(top)) return fail(CTHIP_E_BAD_ARG, "cthip_program_create: %s", ps.err.c_str());
  Program *pg = new Program();
  std::string err;
  if (!build_item(top, pg->item, err)) {
    delete pg;
    return fail(CTHIP_E_BAD_ARG, "cthip_program_create: %s", err.c_str());
  }
  KernelRenderer kr(pg->item);
  if (!kr.render(*pg, err)) {
    delete pg;
    return fail(CTHIP_E_UNSUPPORTED, "cthip_program_create: %s", err.c_str());
  }
  Route r;
  if (match_matmul(pg->item, r)) pg->route = r, pg->route_name = "matmul";
  else if ((r = Route(), match_embedding(pg->item, r))) pg->route = r, pg->route_name = "embedding";
  else if ((r = Route(), match_argmax(pg->item, r))) pg->route = r, pg->route_name = "argmax";
  else if ((r = Route(), match_softmax(pg->item, r))) pg->route = r, pg->route_name = "softmax";
  else if ((r = Route(), match_layernorm(pg->item, r))) pg->route = r, pg->route_name = "layernorm";
  else if ((r = Route(), match_rmsnorm(pg->item, r))) pg->route = r, pg->route_name = "rmsnorm";
  *program = pg;
  return 0;
}

int cthip_program_destroy(void *program) {
  delete (Program *)program;
  return 0;
}

const char *cthip_program_source(const void *program) { return program ? ((const Program *)program)->source.c_str() : ""; }
const char *cthip_program_name(const void *program) { return program ? ((const Program *)program)->item.name.c_str() : ""; }
const char *cthip_program_route(const void *program) { return program ? ((const Program *)program)->route_name.c_str() : ""; }
const char *cthip_program_last_route(const void *program) { return program ? ((const Program *)program)->last_route.c_str() : ""; }

int cthip_program_bind(void *program, void *module) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(program != nullptr && module != nullptr);
  Program *pg = (Program *)program;
  void *fn = nullptr;
  int rc = cthip_get_function(&fn, module, pg->item.name.c_str());
  if (rc) return rc;
  pg->fn = (hipFunction_t)fn;
  return 0;
}

int cthip_program_launch(void *program, void **args, int nargs) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(program != nullptr && (nargs == 0 || args != nullptr));
  Program *pg = (Program *)program;
  const Item &it = pg->item;
  if (nargs != (int)it.globals.size())
    return fail(CTHIP_E_BAD_ARG, "HIP: %s takes %zu arguments, got %d", it.name.c_str(), it.globals.size(), nargs);
  std::map<std::string, long long> env;
  for (int k = 0; k < nargs; k++) {
    const Global &g = it.globals[k];
    if (!args[k]) return fail(CTHIP_E_BAD_ARG, "HIP: %s: argument %s is null", it.name.c_str(), g.id.c_str());
    if (g.pointer) {
      if (!*(void **)args[k]) return fail(CTHIP_E_BAD_ARG, "HIP: please transfer the buffer %s to the device first", g.id.c_str());
      continue;
    }
    long long v = 0;
    if (g.dtype == "int64" || g.dtype == "uint64") v = *(long long *)args[k];
    else if (g.dtype == "int32") v = *(int *)args[k];
    else if (g.dtype == "uint32") v = *(unsigned *)args[k];
    else if (g.dtype == "int16") v = *(short *)args[k];
    else if (g.dtype == "uint16") v = *(unsigned short *)args[k];
    else if (g.dtype == "int8") v = *(signed char *)args[k];
    else if (g.dtype == "uint8" || g.dtype == "bool") v = *(unsigned char *)args[k];
    else continue;  // floating-point scalars do not size anything
    env[g.id] = v;
  }
  if (pg->route.kind != R_NONE && state().render_routes) {
    int rc = 0;
    if (launch_route(*pg, args, env, rc)) return rc;
  }
  if (!pg->fn) return fail(CTHIP_E_STATE, "HIP: %s has not been bound to a compiled module (cthip_program_bind)", it.name.c_str());
  long long total = 1;
  for (const Sx &b : pg->grid_bounds) {
    long long v;
    if (!eval_int(b, env, v)) return fail(CTHIP_E_UNSUPPORTED, "HIP: %s: a loop bound is not an expression of the shape arguments", it.name.c_str());
    total *= v > 0 ? v : 0;
  }
  unsigned grid[3] = {1, 1, 1}, block[3] = {1, 1, 1};
  if (pg->explicit_grid) {
    long long threads = 1;
    for (int q = 0; q < 3; q++) {
      long long g, l;
      if (!eval_int(pg->grid_global[q], env, g) || !eval_int(pg->grid_local[q], env, l))
        return fail(CTHIP_E_UNSUPPORTED, "HIP: %s: a grid size is not an expression of the shape arguments", it.name.c_str());
      if (g < 0 || l < 1 || g > 0x7fffffffll || l > 1024) return fail(CTHIP_E_BAD_ARG, "HIP: %s: grid %lld x %lld along axis %d", it.name.c_str(), g, l, q);
      if (g == 0) return 0;
      grid[q] = (unsigned)g;
      block[q] = (unsigned)l;
      threads *= l;
    }
    if (threads > 1024) return fail(CTHIP_E_BAD_ARG, "HIP: %s: %lld threads per workgroup", it.name.c_str(), threads);
    pg->last_route = "rendered";
    return cthip_launch(pg->fn, grid, block, 0, args, nargs);
  }
  if (pg->parallel) {
    const long long per = pg->rows_per_block;
    const long long nb = (total + per - 1) / per;
    if (nb > 0x7fffffffll) return fail(CTHIP_E_UNSUPPORTED, "HIP: %s: %lld workgroups exceed the grid", it.name.c_str(), nb);
    if (nb == 0) return 0;
    grid[0] = (unsigned)nb;
    block[0] = 256;
  }
  pg->last_route = "rendered";
  return cthip_launch(pg->fn, grid, block, 0, args, nargs);
}

}  // extern "C"
