// An Option_Filter from a pattern over variant names: the hand-written counterpart of the
// learned filter, for variant families too large to explore blindly ("NNN???/*/*" keeps the
// pad, tile and tail choices of GEMM_Options_Pad_Tile and drops its explicit transposes: 120 of
// 960 variants).  The reference has the hook (planning_system.h:14-35) and builds its filters
// from predicates in code; a pattern can come from an input file or across a C ABI.
#pragma once
#include <string>
#include <vector>

#include "planning_system.h"

namespace rtat {

// Glob match: '?' stands for any one character, '*' for any run of characters (also none).
inline bool glob_match(const char* pattern, const char* text) {
  for (; *pattern != '\0'; ++pattern, ++text) {
    if (*pattern == '*') {
      while (pattern[1] == '*') ++pattern;
      for (const char* rest = text;; ++rest) {
        if (glob_match(pattern + 1, rest)) return true;
        if (*rest == '\0') return false;
      }
    }
    if (*text == '\0' || (*pattern != '?' && *pattern != *text)) return false;
  }
  return *text == '\0';
}

// Admits a variant when its name matches one of the comma-separated patterns.  The default
// variant is always admitted: the planner falls back to it when workspace is short.
template <typename Key, typename Opts>
Option_Filter<Key, Opts> pattern_filter(const std::string& patterns) {
  std::vector<std::string> alternatives;
  size_t from = 0;
  for (size_t at; (at = patterns.find(',', from)) != std::string::npos; from = at + 1)
    alternatives.push_back(patterns.substr(from, at - from));
  alternatives.push_back(patterns.substr(from));
  const std::string fallback = std::string(Opts::default_opts());
  return Option_Filter<Key, Opts>([alternatives, fallback](std::pair<Opts, Key> candidate) {
    const std::string name = std::string(candidate.first);
    if (name == fallback) return true;
    for (const std::string& p : alternatives)
      if (glob_match(p.c_str(), name.c_str())) return true;
    return false;
  });
}

}  // namespace rtat
