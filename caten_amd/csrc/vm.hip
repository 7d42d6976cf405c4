// The walk of a compiled node list behind ONE call per forward.
//
// Caten's GraphRuntime steps through a flat list of nodes (runtime-forward / runtime-step,
// source/runtime/runtime.lisp:106-145): `:Allocate` opens or reuses a buffer whose shape is given by numbers or by
// scalar variables (runtime.lisp:228-259), the scalar nodes `:Add :Mul :Neg :Idiv :Mod :Max` compute dynamic shapes
// and strides (runtime.lisp:396-449), and `:JIT_KERNEL` launches one compiled Schedule-Item and returns the arguments
// at its out-positions (source/codegen/runner.lisp:20-32).  The reference runs that walk in compiled Lisp; a host
// that is slower per node than a launch (150 launches of a GPT-2 decode step leave the device idle between them)
// hands the list over once -- slots instead of variable names, programs instead of callers -- and asks for a whole
// forward with one call.  Node kinds beyond these three (views, custom ops) stay with the host's own walk.
//
// Buffers opened by `:Allocate` belong to the node (its pool, as in the reference): the same shape on the next forward
// gets the same storage back with its contents (the KV cache relies on that), another shape gets zero-filled
// storage, as closing the pool and opening a new buffer would give it.  Parameters and inputs are bound from outside (`:Allocate :from`) and never freed here.
//
// Shapes depend on the forward's inputs only, never on a kernel's result, so a forward first evaluates every scalar
// node and opens every buffer, clears all newly opened storage with ONE launch (a decode step re-opens every buffer
// whose shape contains the position: 25 of them for a 12-layer GPT-2), and then issues the kernels back to back.
// (A list in which a variable is written by more than one node is walked strictly in order instead.)
#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <chrono>
#include <map>
#include <string>
#include <vector>

#include "common.h"

namespace cthip {

enum { VM_UNSET = 0, VM_INT = 1, VM_FLOAT = 2, VM_BUF = 3 };
enum { VM_OPND_INT = 0, VM_OPND_FLOAT = 1, VM_OPND_SLOT = 2 };
enum { VM_NODE_SCALAR = 0, VM_NODE_ALLOCATE = 1, VM_NODE_KERNEL = 2 };
enum { VM_ADD = 0, VM_MUL = 1, VM_NEG = 2, VM_IDIV = 3, VM_MOD = 4, VM_MAX = 5 };

struct VmSlot {
  int kind = VM_UNSET;
  long long i = 0;
  double f = 0.0;
  void *ptr = nullptr;
};

struct VmOperand {
  int kind;
  long long i;
  double f;
};

struct VmNode {
  int type = 0, op = 0, out = -1;
  std::vector<VmOperand> in;
  // :Allocate
  int elem_bytes = 0;
  void *pool = nullptr;
  size_t pool_bytes = 0;                 // capacity of the storage behind the pool
  std::vector<long long> pool_shape;
  // :JIT_KERNEL
  void *program = nullptr;
  std::vector<int> dtypes;               // per argument: CTHIP_VM_PTR or the code of a by-value scalar type
  std::vector<int> out_pos, out_slots;   // writes[k] = args[out_pos[k]]
  long long host_ns = 0, calls = 0;      // CTHIP_VM_PROFILE=1: host time spent issuing this node
};

constexpr int kFillRanges = 32;
struct FillRanges {
  void *ptr[kFillRanges];
  unsigned long long n16[kFillRanges];      // 16-byte units
  unsigned first_block[kFillRanges + 1];    // blocks [first_block[r], first_block[r + 1]) clear range r
  int n;
};
constexpr unsigned kFillPerBlock = 256 * 8;  // 16-byte units a block clears

__global__ __launch_bounds__(256) void k_fill_ranges(FillRanges fr) {
  int r = 0;
  while (r + 1 < fr.n && blockIdx.x >= fr.first_block[r + 1]) r++;
  const unsigned long long lo = (unsigned long long)(blockIdx.x - fr.first_block[r]) * kFillPerBlock;
  const unsigned long long hi = lo + kFillPerBlock < fr.n16[r] ? lo + kFillPerBlock : fr.n16[r];
  uint4 *p = (uint4 *)fr.ptr[r];
  const uint4 z = make_uint4(0u, 0u, 0u, 0u);
  for (unsigned long long i = lo + threadIdx.x; i < hi; i += 256) p[i] = z;
}

struct Vm {
  std::vector<VmSlot> slots;
  std::vector<VmNode> nodes;
  std::vector<int> writers;               // per slot: nodes that write it
  bool hoist = true;                      // scalars and buffers first, one fill, then the kernels
  std::vector<std::pair<void *, unsigned long long>> fills;  // newly opened storage of this forward (pointer, 16-byte units)
  std::vector<unsigned long long> cells;  // one 8-byte cell per kernel argument
  std::vector<void *> argv;
  long long launches = 0;
  bool profile = false;                   // CTHIP_VM_PROFILE=1: per-program host time, printed by cthip_vm_destroy
  long long open_ns = 0, runs = 0;        // ... and of the scalar nodes, the buffers and their clearing
};

static bool vm_value(const Vm &vm, const VmOperand &o, VmSlot &v) {
  if (o.kind == VM_OPND_INT) {
    v.kind = VM_INT;
    v.i = o.i;
    return true;
  }
  if (o.kind == VM_OPND_FLOAT) {
    v.kind = VM_FLOAT;
    v.f = o.f;
    return true;
  }
  if (o.i < 0 || o.i >= (long long)vm.slots.size()) return false;
  v = vm.slots[(size_t)o.i];
  return v.kind != VM_UNSET;
}

static long long floordiv(long long a, long long b) {
  long long q = a / b;
  if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
  return q;
}

static int vm_scalar(Vm &vm, int idx, VmNode &n) {
  VmSlot a[8];
  const int cnt = (int)n.in.size();
  bool all_int = true;
  for (int k = 0; k < cnt; k++) {
    if (!vm_value(vm, n.in[(size_t)k], a[k]) || a[k].kind == VM_BUF)
      return fail(CTHIP_E_STATE, "vm: node %d: operand %d of a scalar node is not a number that has been set", idx, k);
    all_int = all_int && a[k].kind == VM_INT;
  }
  auto num = [&](int k) { return a[k].kind == VM_INT ? (double)a[k].i : a[k].f; };
  VmSlot r;
  r.kind = all_int ? VM_INT : VM_FLOAT;
  switch (n.op) {
    case VM_ADD:
      if (all_int) for (int k = 0; k < cnt; k++) r.i += a[k].i;
      else for (int k = 0; k < cnt; k++) r.f += num(k);
      break;
    case VM_MUL:
      r.i = 1;
      r.f = 1.0;
      if (all_int) for (int k = 0; k < cnt; k++) r.i *= a[k].i;
      else for (int k = 0; k < cnt; k++) r.f *= num(k);
      break;
    case VM_NEG:
      if (all_int) r.i = -a[0].i;
      else r.f = -num(0);
      break;
    case VM_IDIV:
    case VM_MOD:
      if (all_int) {
        if (a[1].i == 0) return fail(CTHIP_E_STATE, "vm: node %d: division by zero", idx);
        const long long q = floordiv(a[0].i, a[1].i);
        r.i = n.op == VM_IDIV ? q : a[0].i - q * a[1].i;
      } else {
        if (num(1) == 0.0) return fail(CTHIP_E_STATE, "vm: node %d: division by zero", idx);
        const double q = floor(num(0) / num(1));
        r.f = n.op == VM_IDIV ? q : num(0) - q * num(1);
      }
      break;
    case VM_MAX:
      if (all_int) {
        r.i = a[0].i;
        for (int k = 1; k < cnt; k++) r.i = a[k].i > r.i ? a[k].i : r.i;
      } else {
        r.f = num(0);
        for (int k = 1; k < cnt; k++) r.f = num(k) > r.f ? num(k) : r.f;
      }
      break;
    default: return fail(CTHIP_E_BAD_ARG, "vm: node %d: unknown scalar operation %d", idx, n.op);
  }
  vm.slots[(size_t)n.out] = r;
  return 0;
}

static int vm_allocate(Vm &vm, int idx, VmNode &n) {
  const int nrank = (int)n.in.size();
  long long shape[8], count = 1;
  for (int k = 0; k < nrank; k++) {
    VmSlot v;
    if (!vm_value(vm, n.in[(size_t)k], v) || v.kind != VM_INT || v.i < 0)
      return fail(CTHIP_E_STATE, "vm: node %d: axis %d of an :Allocate is not a non-negative integer that has been set", idx, k);
    shape[k] = v.i;
    if (v.i && count > (1ll << 46) / v.i)  // (a wrapped product would open a small buffer for kernels that believe the shape)
      return fail(CTHIP_E_BAD_ARG, "vm: node %d: an :Allocate of more than 2^46 elements", idx);
    count *= v.i;
  }
  bool same = n.pool != nullptr && (int)n.pool_shape.size() == nrank;
  for (int k = 0; same && k < nrank; k++) same = n.pool_shape[(size_t)k] == shape[k];
  if (!same) {
    // Another shape: the reference closes the pool and opens a zero-filled buffer.  Here the storage stays when it
    // is large enough (a buffer whose shape contains the position grows by a row a step; a new block from the
    // driver every few steps costs more than the whole forward) and is cleared like a newly opened one; a buffer
    // that has to grow gets half as much again.
    const size_t bytes = (((size_t)(count > 0 ? count : 1) * (size_t)n.elem_bytes) + 15) & ~(size_t)15;
    if (!n.pool || bytes > n.pool_bytes) {
      const size_t want = n.pool ? bytes + bytes / 2 : bytes;
      if (n.pool) cthip_free(n.pool);
      n.pool = nullptr;
      n.pool_bytes = 0;
      int rc = alloc_scratch(&n.pool, want);
      if (rc) return rc;
      n.pool_bytes = want;
    }
    vm.fills.push_back({n.pool, (unsigned long long)(bytes / 16)});
    n.pool_shape.assign(shape, shape + nrank);
  }
  VmSlot &s = vm.slots[(size_t)n.out];
  s.kind = VM_BUF;
  s.ptr = n.pool;
  return 0;
}

static int vm_flush_fills(Vm &vm) {
  size_t at = 0;
  while (at < vm.fills.size()) {
    FillRanges fr;
    fr.n = 0;
    fr.first_block[0] = 0;
    while (at < vm.fills.size() && fr.n < kFillRanges) {
      const unsigned long long blocks = (vm.fills[at].second + kFillPerBlock - 1) / kFillPerBlock;
      if (fr.first_block[fr.n] + blocks > 0x7fffffffull) {
        if (fr.n) break;  // a launch of its own
        return fail(CTHIP_E_UNSUPPORTED, "vm: a buffer of %llu bytes is too large to clear in one launch", vm.fills[at].second * 16);
      }
      fr.ptr[fr.n] = vm.fills[at].first;
      fr.n16[fr.n] = vm.fills[at].second;
      fr.first_block[fr.n + 1] = fr.first_block[fr.n] + (unsigned)blocks;
      fr.n++;
      at++;
    }
    hipLaunchKernelGGL(k_fill_ranges, dim3(fr.first_block[fr.n]), dim3(256), 0, state().stream, fr);
    CTHIP_LAUNCH_CHECK();
  }
  vm.fills.clear();
  return 0;
}

// a number as the declared type of a by-value kernel argument (coerce-dtyped-buffer, source/codegen/helpers.lisp:118-125)
static bool vm_store_scalar(int code, const VmSlot &v, void *cell) {
  const bool is_int = v.kind == VM_INT;
  const double f = is_int ? (double)v.i : v.f;
  const long long i = is_int ? v.i : (long long)v.f;
  switch (code) {
    case CTHIP_VM_BOOL: *(unsigned char *)cell = is_int ? (v.i != 0) : (v.f != 0.0); return true;
    case CTHIP_VM_F64: *(double *)cell = f; return true;
    case CTHIP_VM_F32: *(float *)cell = (float)f; return true;
    case CTHIP_VM_U64: *(unsigned long long *)cell = (unsigned long long)i; return true;
    case CTHIP_VM_I64: *(long long *)cell = i; return true;
    case CTHIP_VM_U32: *(unsigned *)cell = (unsigned)i; return true;
    case CTHIP_VM_I32: *(int *)cell = (int)i; return true;
    case CTHIP_VM_U16: *(unsigned short *)cell = (unsigned short)i; return true;
    case CTHIP_VM_I16: *(short *)cell = (short)i; return true;
    case CTHIP_VM_U8: *(unsigned char *)cell = (unsigned char)i; return true;
    case CTHIP_VM_I8: *(signed char *)cell = (signed char)i; return true;
    default: return false;
  }
}

static int vm_kernel(Vm &vm, int idx, VmNode &n) {
  const int nargs = (int)n.in.size();
  if ((int)vm.cells.size() < nargs) {
    vm.cells.resize((size_t)nargs);
    vm.argv.resize((size_t)nargs);
  }
  for (int k = 0; k < nargs; k++) {
    VmSlot v;
    if (!vm_value(vm, n.in[(size_t)k], v)) return fail(CTHIP_E_STATE, "vm: node %d: argument %d has not been set", idx, k);
    void *cell = &vm.cells[(size_t)k];
    vm.cells[(size_t)k] = 0;
    if (n.dtypes[(size_t)k] == CTHIP_VM_PTR) {
      if (v.kind != VM_BUF || !v.ptr) return fail(CTHIP_E_STATE, "vm: node %d: argument %d must be a device buffer", idx, k);
      *(void **)cell = v.ptr;
    } else {
      if (v.kind == VM_BUF || !vm_store_scalar(n.dtypes[(size_t)k], v, cell))
        return fail(CTHIP_E_STATE, "vm: node %d: argument %d must be a number of type code %d", idx, k, n.dtypes[(size_t)k]);
    }
    vm.argv[(size_t)k] = cell;
  }
  int rc;
  if (vm.profile) {
    const auto t0 = std::chrono::steady_clock::now();
    rc = cthip_program_launch(n.program, vm.argv.data(), nargs);
    // (a node's first launch pays one-time costs -- code loading, packing of a weight matrix -- and is left out)
    if (n.calls++) n.host_ns += std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
  } else {
    rc = cthip_program_launch(n.program, vm.argv.data(), nargs);
  }
  if (rc) return rc;
  vm.launches++;
  for (size_t k = 0; k < n.out_pos.size(); k++) {
    VmSlot v;
    vm_value(vm, n.in[(size_t)n.out_pos[k]], v);
    vm.slots[(size_t)n.out_slots[k]] = v;
  }
  return 0;
}

}  // namespace cthip

using namespace cthip;

extern "C" {

int cthip_vm_create(void **vm, int n_slots) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(vm != nullptr && n_slots > 0);
  Vm *v = new Vm();
  v->slots.resize((size_t)n_slots);
  v->writers.assign((size_t)n_slots, 0);
  const char *prof = getenv("CTHIP_VM_PROFILE");
  v->profile = prof && prof[0] == '1';
  *vm = v;
  return 0;
}

int cthip_vm_destroy(void *vm) {
  if (!vm) return 0;
  Vm *v = (Vm *)vm;
  if (state().inited) (void)hipStreamSynchronize(state().stream);
  if (v->profile) {  // host time per program, as PROFILE=1 prints per kernel in the reference (source/codegen/runner.lisp:7-31)
    std::map<std::string, std::pair<long long, long long>> by_name;
    for (VmNode &n : v->nodes)
      if (n.type == VM_NODE_KERNEL && n.calls > 1) {
        auto &e = by_name[std::string(cthip_program_name(n.program)) + " -> " + cthip_program_last_route(n.program)];
        e.first += n.host_ns;
        e.second += n.calls - 1;
      }
    if (v->runs > 1)
      fprintf(stderr, "[cthip vm] scalar nodes, buffers and their clearing: %.2f us of host time per forward\n",
              (double)v->open_ns / (double)(v->runs - 1) * 1e-3);
    for (const auto &kv : by_name)
      fprintf(stderr, "[cthip vm] %-48s %8lld launches  %7.2f us of host time each\n", kv.first.c_str(), kv.second.second,
              (double)kv.second.first / (double)kv.second.second * 1e-3);
  }
  for (VmNode &n : v->nodes)
    if (n.pool) cthip_free(n.pool);
  delete v;
  return 0;
}

static int vm_operands(Vm *v, int n, const int *kinds, const long long *ivals, const double *fvals, std::vector<VmOperand> &out) {
  for (int k = 0; k < n; k++) {
    VmOperand o = {kinds[k], ivals ? ivals[k] : 0, fvals ? fvals[k] : 0.0};
    if (o.kind < VM_OPND_INT || o.kind > VM_OPND_SLOT) return fail(CTHIP_E_BAD_ARG, "vm: operand %d has kind %d", k, o.kind);
    if (o.kind == VM_OPND_SLOT && (o.i < 0 || o.i >= (long long)v->slots.size()))
      return fail(CTHIP_E_BAD_ARG, "vm: operand %d names slot %lld of %zu", k, o.i, v->slots.size());
    out.push_back(o);
  }
  return 0;
}

int cthip_vm_add_scalar(void *vm, int op, int out, int n_in, const int *kinds, const long long *ivals, const double *fvals) {
  CTHIP_ARG(vm != nullptr && kinds != nullptr && n_in >= 1 && n_in <= 8);
  Vm *v = (Vm *)vm;
  CTHIP_ARG(out >= 0 && out < (int)v->slots.size() && op >= VM_ADD && op <= VM_MAX);
  if ((op == VM_NEG && n_in != 1) || ((op == VM_IDIV || op == VM_MOD) && n_in != 2))
    return fail(CTHIP_E_BAD_ARG, "vm: scalar operation %d with %d operands", op, n_in);
  VmNode n;
  n.type = VM_NODE_SCALAR;
  n.op = op;
  n.out = out;
  int rc = vm_operands(v, n_in, kinds, ivals, fvals, n.in);
  if (rc) return rc;
  v->nodes.push_back(n);
  if (++v->writers[(size_t)out] > 1) v->hoist = false;
  return 0;
}

int cthip_vm_add_allocate(void *vm, int out, int elem_bytes, int nrank, const int *kinds, const long long *ivals) {
  CTHIP_ARG(vm != nullptr && nrank >= 0 && nrank <= 8 && (nrank == 0 || kinds != nullptr) && elem_bytes > 0 && elem_bytes <= 8);
  Vm *v = (Vm *)vm;
  CTHIP_ARG(out >= 0 && out < (int)v->slots.size());
  VmNode n;
  n.type = VM_NODE_ALLOCATE;
  n.out = out;
  n.elem_bytes = elem_bytes;
  int rc = vm_operands(v, nrank, kinds, ivals, nullptr, n.in);
  if (rc) return rc;
  for (const VmOperand &o : n.in)
    if (o.kind == VM_OPND_FLOAT) return fail(CTHIP_E_BAD_ARG, "vm: an :Allocate axis is a floating-point literal");
  v->nodes.push_back(n);
  if (++v->writers[(size_t)out] > 1) v->hoist = false;
  return 0;
}

int cthip_vm_add_kernel(void *vm, void *program, int nargs, const int *kinds, const long long *ivals, const double *fvals,
                        const int *dtypes, int n_out, const int *out_positions, const int *out_slots) {
  CTHIP_ARG(vm != nullptr && program != nullptr && nargs >= 0 && (nargs == 0 || (kinds != nullptr && dtypes != nullptr)));
  CTHIP_ARG(n_out >= 0 && (n_out == 0 || (out_positions != nullptr && out_slots != nullptr)));
  Vm *v = (Vm *)vm;
  VmNode n;
  n.type = VM_NODE_KERNEL;
  n.program = program;
  int rc = vm_operands(v, nargs, kinds, ivals, fvals, n.in);
  if (rc) return rc;
  for (int k = 0; k < nargs; k++) {
    if (dtypes[k] < CTHIP_VM_PTR || dtypes[k] > CTHIP_VM_I8) return fail(CTHIP_E_BAD_ARG, "vm: argument %d has type code %d", k, dtypes[k]);
    n.dtypes.push_back(dtypes[k]);
  }
  for (int k = 0; k < n_out; k++) {
    if (out_positions[k] < 0 || out_positions[k] >= nargs || out_slots[k] < 0 || out_slots[k] >= (int)v->slots.size())
      return fail(CTHIP_E_BAD_ARG, "vm: output %d is argument %d into slot %d", k, out_positions[k], out_slots[k]);
    n.out_pos.push_back(out_positions[k]);
    n.out_slots.push_back(out_slots[k]);
    // a result under the name of the argument it is stored in writes nothing new
    const VmOperand &src = n.in[(size_t)out_positions[k]];
    if (!(src.kind == VM_OPND_SLOT && src.i == out_slots[k]) && ++v->writers[(size_t)out_slots[k]] > 1) v->hoist = false;
  }
  v->nodes.push_back(n);
  return 0;
}

int cthip_vm_set_int(void *vm, int slot, long long value) {
  CTHIP_ARG(vm != nullptr);
  Vm *v = (Vm *)vm;
  CTHIP_ARG(slot >= 0 && slot < (int)v->slots.size());
  VmSlot s;
  s.kind = VM_INT;
  s.i = value;
  v->slots[(size_t)slot] = s;
  return 0;
}

int cthip_vm_set_float(void *vm, int slot, double value) {
  CTHIP_ARG(vm != nullptr);
  Vm *v = (Vm *)vm;
  CTHIP_ARG(slot >= 0 && slot < (int)v->slots.size());
  VmSlot s;
  s.kind = VM_FLOAT;
  s.f = value;
  v->slots[(size_t)slot] = s;
  return 0;
}

int cthip_vm_set_buffer(void *vm, int slot, void *device_ptr) {
  CTHIP_ARG(vm != nullptr && device_ptr != nullptr);
  Vm *v = (Vm *)vm;
  CTHIP_ARG(slot >= 0 && slot < (int)v->slots.size());
  VmSlot s;
  s.kind = VM_BUF;
  s.ptr = device_ptr;
  v->slots[(size_t)slot] = s;
  return 0;
}

int cthip_vm_run(void *vm) {
  CTHIP_REQUIRE_INIT();
  CTHIP_ARG(vm != nullptr);
  Vm *v = (Vm *)vm;
  int rc = 0;
  v->fills.clear();
  if (v->hoist) {
    const auto t0 = std::chrono::steady_clock::now();
    for (size_t k = 0; k < v->nodes.size() && !rc; k++) {
      VmNode &n = v->nodes[k];
      if (n.type == VM_NODE_SCALAR) rc = vm_scalar(*v, (int)k, n);
      else if (n.type == VM_NODE_ALLOCATE) rc = vm_allocate(*v, (int)k, n);
    }
    {  // also after a failure: storage that was opened is cleared, a later forward finds its shape unchanged
      const int rc2 = vm_flush_fills(*v);
      if (!rc) rc = rc2;
    }
    if (v->profile && v->runs++)  // (the first forward opens everything)
      v->open_ns += std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - t0).count();
    for (size_t k = 0; k < v->nodes.size() && !rc; k++)
      if (v->nodes[k].type == VM_NODE_KERNEL) rc = vm_kernel(*v, (int)k, v->nodes[k]);
    return rc;
  }
  for (size_t k = 0; k < v->nodes.size() && !rc; k++) {
    VmNode &n = v->nodes[k];
    if (n.type == VM_NODE_SCALAR) rc = vm_scalar(*v, (int)k, n);
    else if (n.type == VM_NODE_ALLOCATE) {
      rc = vm_allocate(*v, (int)k, n);
      if (!rc) rc = vm_flush_fills(*v);
    } else rc = vm_kernel(*v, (int)k, n);
  }
  return rc;
}

int cthip_vm_get(const void *vm, int slot, int *kind, long long *ivalue, double *fvalue, void **device_ptr) {
  CTHIP_ARG(vm != nullptr && kind != nullptr);
  const Vm *v = (const Vm *)vm;
  CTHIP_ARG(slot >= 0 && slot < (int)v->slots.size());
  const VmSlot &s = v->slots[(size_t)slot];
  *kind = s.kind;
  if (ivalue) *ivalue = s.i;
  if (fvalue) *fvalue = s.f;
  if (device_ptr) *device_ptr = s.ptr;
  return 0;
}

long long cthip_vm_launches(const void *vm) { return vm ? ((const Vm *)vm)->launches : -1; }

}  // extern "C"
