// Problem keys and variant descriptors are identified by their spelling: the text is what
// they are ordered by in the planner's maps, what they print as, and (for variants) what a
// stream reader parses.  A type states its spelling once and inherits the rest from here.
#pragma once
#include <istream>
#include <ostream>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

namespace rtat {

// D provides `std::string text() const`.  Ordering is lexicographic on the text — the same
// order the reference's keys and variants have (e.g. gemm.cpp:18-20), so maps and the JSON
// reports built from them iterate alike.
template <class D>
struct Spelled {
  operator std::string() const { return static_cast<const D&>(*this).text(); }
  friend bool operator<(const D& a, const D& b) { return a.text() < b.text(); }
  friend std::ostream& operator<<(std::ostream& os, const D& d) { return os << d.text(); }
};

// A problem key: its fields never change after construction, so the spelling is built once
// and every later comparison is a plain string compare without allocation.  D passes the
// finished text to the constructor.
template <class D>
class Spelled_Once {
  std::string label;

 protected:
  explicit Spelled_Once(std::string text) : label(std::move(text)) {}

 public:
  const std::string& text() const { return label; }
  operator std::string() const { return label; }
  friend bool operator<(const D& a, const D& b) { return a.text() < b.text(); }
  friend std::ostream& operator<<(std::ostream& os, const D& d) { return os << d.text(); }
};

// A variant made of independent switches (BLAS_Op, Pad_Op, Bool_Op, Tile_Op ...).  D provides
// `auto switches()` / `auto switches() const`: a std::tie of its switch members in spelling
// order.  From that follow
//   * text():       the switches' letters back to back ("TNN", "FT", "NNTNPN");
//   * enumerate():  every setting, first switch slowest ("NNN NNT NTN ...");
//   * spell_into(): the inverse of text(), false when the text has the wrong length.
// Types with a different spelling (a separator, a multi-letter switch) override text() and
// spell_into() and keep the rest.
template <class D>
struct Switch_Variant : Spelled<D> {
  static D default_opts() { return D(); }

  std::string text() const {
    std::string out;
    std::apply([&](const auto&... sw) { ((out += std::string(sw)), ...); },
               static_cast<const D&>(*this).switches());
    return out;
  }

  static std::vector<D> enumerate() {
    std::vector<D> settings{D()};
    vary<0>(settings);
    return settings;
  }

  // Sets every switch from one letter each.  A wrong length leaves `d` alone and returns
  // false; a letter that spells nothing throws, as the switch types themselves do.
  static bool spell_into(D& d, const std::string& text) {
    constexpr size_t count = std::tuple_size_v<decltype(std::declval<D&>().switches())>;
    if (text.size() != count) return false;
    D fresh;
    size_t at = 0;
    std::apply(
        [&](auto&... sw) {
          ((sw = std::remove_reference_t<decltype(sw)>(text[at++])), ...);
        },
        fresh.switches());
    d = fresh;
    return true;
  }

  friend std::istream& operator>>(std::istream& is, D& d) {
    std::string word;
    is >> word;
    if (!D::spell_into(d, word)) is.setstate(std::ios::failbit);
    return is;
  }

 private:
  template <size_t I>
  static void vary(std::vector<D>& settings) {
    if constexpr (I < std::tuple_size_v<decltype(std::declval<D&>().switches())>) {
      using Switch = std::remove_reference_t<decltype(std::get<I>(std::declval<D&>().switches()))>;
      std::vector<D> widened;
      for (const D& d : settings)
        for (const Switch& value : Switch::enumerate()) {
          D e = d;
          std::get<I>(e.switches()) = value;
          widened.push_back(e);
        }
      settings.swap(widened);
      vary<I + 1>(settings);
    }
  }
};

}  // namespace rtat
