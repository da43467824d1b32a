// Flop count of the dynamics oracle — TEST / MEASUREMENT INFRASTRUCTURE, never part of the product path.
//
// Compiles ks_dyn_oracle.c a third time with REAL = a scalar type whose +, -, *, / (and their assigning forms), sqrt, exp,
// log, sin, cos, pow, fmin, fmax count one floating-point operation each; comparisons, negation, copies and integer work
// count nothing.  The arithmetic itself is done in double, so the counted run takes the same branches (contacts, solver
// iterations, line-search steps) as the float64 oracle.  Entry points carry the suffix _cnt; the counter is one global,
// so run it with one thread.
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

static double g_flops = 0;

struct Counted {
  double v;
  Counted() = default;
  Counted(double x) : v(x) {}
  Counted(int x) : v(x) {}
  explicit operator double() const { return v; }
  explicit operator float() const { return (float)v; }
  explicit operator int() const { return (int)v; }
};
static_assert(sizeof(Counted) == sizeof(double), "the counted data block has the layout of the float64 one");

#define KS_BIN(op)                                                                                  \
  inline Counted operator op(Counted a, Counted b) { g_flops += 1; return Counted(a.v op b.v); }     \
  inline Counted operator op(Counted a, double b) { g_flops += 1; return Counted(a.v op b); }        \
  inline Counted operator op(double a, Counted b) { g_flops += 1; return Counted(a op b.v); }        \
  inline Counted operator op(Counted a, int b) { g_flops += 1; return Counted(a.v op b); }           \
  inline Counted operator op(int a, Counted b) { g_flops += 1; return Counted(a op b.v); }
KS_BIN(+) KS_BIN(-) KS_BIN(*) KS_BIN(/)
#define KS_ASSIGN(op, bop)                                                                          \
  inline Counted& operator op(Counted& a, Counted b) { g_flops += 1; a.v = a.v bop b.v; return a; }  \
  inline Counted& operator op(Counted& a, double b) { g_flops += 1; a.v = a.v bop b; return a; }
KS_ASSIGN(+=, +) KS_ASSIGN(-=, -) KS_ASSIGN(*=, *) KS_ASSIGN(/=, /)
inline Counted operator-(Counted a) { return Counted(-a.v); }
#define KS_CMP(op)                                                   \
  inline bool operator op(Counted a, Counted b) { return a.v op b.v; } \
  inline bool operator op(Counted a, double b) { return a.v op b; }    \
  inline bool operator op(double a, Counted b) { return a op b.v; }    \
  inline bool operator op(Counted a, int b) { return a.v op b; }       \
  inline bool operator op(int a, Counted b) { return a op b.v; }
KS_CMP(<) KS_CMP(>) KS_CMP(<=) KS_CMP(>=) KS_CMP(==) KS_CMP(!=)
#define KS_FUN1(f) \
  inline Counted f(Counted a) { g_flops += 1; return Counted(::f(a.v)); }
KS_FUN1(sqrt) KS_FUN1(exp) KS_FUN1(log) KS_FUN1(sin) KS_FUN1(cos) KS_FUN1(tanh)
inline Counted fabs(Counted a) { return Counted(::fabs(a.v)); }
inline Counted floor(Counted a) { return Counted(::floor(a.v)); }
inline Counted pow(Counted a, Counted b) { g_flops += 1; return Counted(::pow(a.v, b.v)); }
inline Counted pow(Counted a, double b) { g_flops += 1; return Counted(::pow(a.v, b)); }
inline Counted fmax(Counted a, Counted b) { g_flops += 1; return Counted(::fmax(a.v, b.v)); }
inline Counted fmin(Counted a, Counted b) { g_flops += 1; return Counted(::fmin(a.v, b.v)); }
inline Counted atan2(Counted a, Counted b) { g_flops += 1; return Counted(::atan2(a.v, b.v)); }

#define REAL Counted
#define SUF _cnt
extern "C" {
#include "ks_dyn_oracle.c"
double ksor_flops(void) { return g_flops; }
void ksor_flops_reset(void) { g_flops = 0; }
}
