// Option atoms the variant descriptors are made of (reference src/methods/base_options.h):
// two-valued switches with a one-letter spelling used in variant strings and plan JSON.
#pragma once
#include <rtat_native.h>

#include <stdexcept>
#include <string>
#include <vector>

namespace rtat {

namespace detail {
// A switch with values {off, on} spelled by the two letters of Spelling.
template <class Spelling>
struct Two_Valued {
  static bool parse(const std::string& s) {
    if (s.size() == 1 && s[0] == Spelling::off) return false;
    if (s.size() == 1 && s[0] == Spelling::on) return true;
    throw std::runtime_error(std::string("Invalid ") + Spelling::what + " string " + s);
  }
  static std::string spell(bool on) { return std::string(1, on ? Spelling::on : Spelling::off); }
};
struct Op_Spelling { static constexpr char off = 'N', on = 'T'; static constexpr const char* what = "BLAS_Op"; };
struct Pad_Spelling { static constexpr char off = 'N', on = 'P'; static constexpr const char* what = "Pad_Op"; };
struct Bool_Spelling { static constexpr char off = 'F', on = 'T'; static constexpr const char* what = "bool op"; };
}  // namespace detail

// "N" / "T": leave an operand as it is, or materialise its transpose first.
class BLAS_Op {
 public:
  enum _BLAS_Op { NOTRANS, TRANS };
  _BLAS_Op op = NOTRANS;

  BLAS_Op() = default;
  BLAS_Op(_BLAS_Op op) : op(op) {}
  BLAS_Op(const std::string& s) : op(detail::Two_Valued<detail::Op_Spelling>::parse(s) ? TRANS : NOTRANS) {}
  BLAS_Op(char c) : BLAS_Op(std::string(1, c)) {}
  bool operator==(_BLAS_Op o) const { return op == o; }
  BLAS_Op operator!() const { return BLAS_Op(op == TRANS ? NOTRANS : TRANS); }
  operator std::string() const { return detail::Two_Valued<detail::Op_Spelling>::spell(op == TRANS); }
  static std::vector<BLAS_Op> enumerate() { return {BLAS_Op(NOTRANS), BLAS_Op(TRANS)}; }
};

// "N" / "P": leave an operand's leading dimension, or copy it to a padded one first.
class Pad_Op {
 public:
  enum _Pad_Op { NOPAD, PAD };
  _Pad_Op op = NOPAD;

  Pad_Op() = default;
  Pad_Op(_Pad_Op op) : op(op) {}
  Pad_Op(const std::string& s) : op(detail::Two_Valued<detail::Pad_Spelling>::parse(s) ? PAD : NOPAD) {}
  Pad_Op(char c) : Pad_Op(std::string(1, c)) {}
  bool operator==(_Pad_Op o) const { return op == o; }
  Pad_Op operator!() const { return Pad_Op(op == PAD ? NOPAD : PAD); }
  operator std::string() const { return detail::Two_Valued<detail::Pad_Spelling>::spell(op == PAD); }
  static std::vector<Pad_Op> enumerate() { return {Pad_Op(NOPAD), Pad_Op(PAD)}; }
};

// "F" / "T".  (The reference builds these from a char in its stream readers, which always
// yields true — syrk.cpp:64-65, trsm.cpp:65-66; the char constructor here parses the letter.)
class Bool_Op {
 public:
  bool op = false;

  Bool_Op() = default;
  Bool_Op(bool op) : op(op) {}
  Bool_Op(const std::string& s) : op(detail::Two_Valued<detail::Bool_Spelling>::parse(s)) {}
  Bool_Op(const char* s) : Bool_Op(std::string(s)) {}
  Bool_Op(char c) : Bool_Op(std::string(1, c)) {}
  operator bool() const { return op; }
  Bool_Op operator!() const { return Bool_Op(!op); }
  operator std::string() const { return detail::Two_Valued<detail::Bool_Spelling>::spell(op); }
  static std::vector<Bool_Op> enumerate() { return {Bool_Op(false), Bool_Op(true)}; }
};

// A two-valued switch with a third spelling, 'X'.
//   off:  the result is not transposed;
//   on:   the reference's tree: the transposed result is formed in scratch and a second
//         launch adds it back transposed;
//   'X':  "transposed by the kernel itself, in one launch, without scratch".  The kernels of
//         this library take every operand in either orientation (an op flag selects how a panel
//         is loaded, not a different algorithm; the MFMAs are issued so that the accumulators'
//         lanes run along the caller's contiguous dimension whichever way the product is
//         posed; the panel solve loads and stores its slab transposed for a right-hand system),
//         so that form IS the plain call: 'X' builds the tree of `off`.  It can be asked for by
//         name and is kept in plan files, but it is not enumerated: a planner that tried both
//         would time the same launch twice.
namespace detail {
template <class Spelling>
struct Three_Valued {
  enum Value { OFF = 0, ON = 1, FUSED = 2 };
  static Value parse(const std::string& s) {
    if (s.size() == 1 && s[0] == Spelling::off) return OFF;
    if (s.size() == 1 && s[0] == Spelling::on) return ON;
    if (s.size() == 1 && s[0] == 'X') return FUSED;
    throw std::runtime_error(std::string("Invalid fused ") + Spelling::what + " string " + s);
  }
  static std::string spell(Value v) {
    return std::string(1, v == FUSED ? 'X' : v == ON ? Spelling::on : Spelling::off);
  }
};
}  // namespace detail

template <class Spelling>
class Fusable_Op {
  using Codec = detail::Three_Valued<Spelling>;

 public:
  using Value = typename Codec::Value;
  static constexpr Value OFF = Codec::OFF, ON = Codec::ON, FUSED = Codec::FUSED;
  Value op = OFF;

  Fusable_Op() = default;
  Fusable_Op(Value v) : op(v) {}
  Fusable_Op(const std::string& s) : op(Codec::parse(s)) {}
  Fusable_Op(const char* s) : Fusable_Op(std::string(s)) {}
  Fusable_Op(char c) : Fusable_Op(std::string(1, c)) {}
  bool operator==(Value v) const { return op == v; }
  operator std::string() const { return Codec::spell(op); }
  // FUSED builds the tree of OFF, so a planner that tried both would time one launch twice.
  static std::vector<Fusable_Op> enumerate() { return {Fusable_Op(OFF), Fusable_Op(ON)}; }
};
using Fusable_Trans_Op = Fusable_Op<detail::Op_Spelling>;   // "N" / "T" / "X"
using Fusable_Bool_Op = Fusable_Op<detail::Bool_Spelling>;  // "F" / "T" / "X"

// Switches whose values have names of several letters (kernel options).  In a variant's text
// each is set off by a slash: "NNN/128x64", "FF/auto/split/1024".  One class per option; the
// names come from the library (rtat_gemm_variant_name and friends), and the first value, id 0,
// is always "auto": the library's own choice, which is what the default variant runs.
namespace detail {
template <const char* (*Name)(int)>
class Named_Op {
 public:
  static constexpr bool named = true;
  int id = 0;
  Named_Op() = default;
  Named_Op(int id) : id(id) {
    if (Name(id) == nullptr) throw std::runtime_error("Invalid kernel option id " + std::to_string(id));
  }
  Named_Op(const std::string& name) {
    for (int v = 0; Name(v) != nullptr; ++v)
      if (name == Name(v)) {
        id = v;
        return;
      }
    throw std::runtime_error("Invalid kernel option string " + name);
  }
  Named_Op(const char* name) : Named_Op(std::string(name)) {}
  operator std::string() const { return Name(id); }
  bool operator==(const Named_Op& o) const { return id == o.id; }
};
}  // namespace detail

// Macro-tile shape of the DGEMM core a GEMM / SYRK / TRSM call runs on: "auto", "256x128",
// "128x128", "128x64", "64x64".
class Tile_Op : public detail::Named_Op<&rtat_gemm_variant_name> {
 public:
  using Named_Op::Named_Op;
  static std::vector<Tile_Op> enumerate();
};
// What a launch does with the tiles left over after its last full round: "auto", "whole"
// (every tile by one workgroup), "split" (leftover tiles cut along K).
class Tail_Op : public detail::Named_Op<&rtat_tail_mode_name> {
 public:
  using Named_Op::Named_Op;
  static std::vector<Tail_Op> enumerate();
};
// Rows per launch of the TRSM panel solve: "auto", "512", "1024".
class Panel_Op : public detail::Named_Op<&rtat_trsm_panel_name> {
 public:
  using Named_Op::Named_Op;
  static std::vector<Panel_Op> enumerate();
};

}  // namespace rtat
