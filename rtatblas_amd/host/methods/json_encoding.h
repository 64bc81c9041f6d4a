// JSON codecs of the problem keys and variant descriptors — the plan-file vocabulary.
// Field names and string values are those of the reference (src/methods/json_encoding.h);
// the value type is rtat::Json (json/mini_json.h) instead of nlohmann::json.
#pragma once
#include <mini_json.h>

#include "gemm.h"
#include "syrk.h"
#include "trsm.h"

namespace rtat {

template <typename T>
T from_json(const Json&);

namespace detail {
inline std::string str(const Json& j, const char* key) { return j[key].get<std::string>(); }
}

// {"transA","transB" in "N"/"T", "m","n","k"}
inline Json to_json(const GEMM_Key& key) {
  Json j;
  j["transA"] = std::string(key.transa);
  j["transB"] = std::string(key.transb);
  j["m"] = key.m;
  j["n"] = key.n;
  j["k"] = key.k;
  return j;
}
template <>
inline GEMM_Key from_json<GEMM_Key>(const Json& j) {
  return GEMM_Key(BLAS_Operation(detail::str(j, "transA")), BLAS_Operation(detail::str(j, "transB")),
                  j["m"].get<int>(), j["k"].get<int>(), j["n"].get<int>());
}

// {"transA","transB","transC" in "N"/"T"}
inline Json to_json(const GEMM_Options& o) {
  Json j;
  j["transA"] = std::string(o.transa);
  j["transB"] = std::string(o.transb);
  j["transC"] = std::string(o.transc);
  return j;
}
template <>
inline GEMM_Options from_json<GEMM_Options>(const Json& j) {
  return GEMM_Options(BLAS_Op(detail::str(j, "transA")), BLAS_Op(detail::str(j, "transB")),
                      BLAS_Op(detail::str(j, "transC")));
}

// ... plus {"padA","padB","padC" in "N"/"P"}
inline Json to_json(const GEMM_Options_Pad& o) {
  Json j;
  j["transA"] = std::string(o.transa);
  j["transB"] = std::string(o.transb);
  j["transC"] = std::string(o.transc);
  j["padA"] = std::string(o.pada);
  j["padB"] = std::string(o.padb);
  j["padC"] = std::string(o.padc);
  return j;
}
template <>
inline GEMM_Options_Pad from_json<GEMM_Options_Pad>(const Json& j) {
  return GEMM_Options_Pad(BLAS_Op(detail::str(j, "transA")), Pad_Op(detail::str(j, "padA")),
                          BLAS_Op(detail::str(j, "transB")), Pad_Op(detail::str(j, "padB")),
                          BLAS_Op(detail::str(j, "transC")), Pad_Op(detail::str(j, "padC")));
}

// ... plus {"tile": "256x128" | "128x128" | "128x64" | "64x64" | "auto"}
inline Json to_json(const GEMM_Options_Tile& o) {
  Json j;
  j["transA"] = std::string(o.transa);
  j["transB"] = std::string(o.transb);
  j["transC"] = std::string(o.transc);
  j["tile"] = std::string(o.tile);
  return j;
}
template <>
inline GEMM_Options_Tile from_json<GEMM_Options_Tile>(const Json& j) {
  return GEMM_Options_Tile(BLAS_Op(detail::str(j, "transA")), BLAS_Op(detail::str(j, "transB")),
                           BLAS_Op(detail::str(j, "transC")), Tile_Op(detail::str(j, "tile")));
}

// GEMM_Options_Pad's fields plus {"tile", "tail": "auto" | "whole" | "split"}
inline Json to_json(const GEMM_Options_Pad_Tile& o) {
  Json j;
  j["transA"] = std::string(o.transa);
  j["transB"] = std::string(o.transb);
  j["transC"] = std::string(o.transc);
  j["padA"] = std::string(o.pada);
  j["padB"] = std::string(o.padb);
  j["padC"] = std::string(o.padc);
  j["tile"] = std::string(o.tile);
  j["tail"] = std::string(o.tail);
  return j;
}
template <>
inline GEMM_Options_Pad_Tile from_json<GEMM_Options_Pad_Tile>(const Json& j) {
  return GEMM_Options_Pad_Tile(
      BLAS_Op(detail::str(j, "transA")), BLAS_Op(detail::str(j, "transB")),
      BLAS_Op(detail::str(j, "transC")), Pad_Op(detail::str(j, "padA")),
      Pad_Op(detail::str(j, "padB")), Pad_Op(detail::str(j, "padC")),
      Tile_Op(detail::str(j, "tile")), Tail_Op(detail::str(j, "tail")));
}

// GEMM_Options' fields with "transC" in "N"/"T"/"X"
inline Json to_json(const GEMM_Options_Fused& o) {
  Json j;
  j["transA"] = std::string(o.transa);
  j["transB"] = std::string(o.transb);
  j["transC"] = std::string(o.transc);
  return j;
}
template <>
inline GEMM_Options_Fused from_json<GEMM_Options_Fused>(const Json& j) {
  return GEMM_Options_Fused(BLAS_Op(detail::str(j, "transA")), BLAS_Op(detail::str(j, "transB")),
                            Fusable_Trans_Op(detail::str(j, "transC")));
}

// {"uplo" in "Lower"/"Upper", "trans" in "N"/"T", "n","k"}
inline Json to_json(const SYRK_Key& key) {
  Json j;
  j["uplo"] = std::string(key.uplo);
  j["trans"] = std::string(key.trans);
  j["n"] = key.n;
  j["k"] = key.k;
  return j;
}
template <>
inline SYRK_Key from_json<SYRK_Key>(const Json& j) {
  return SYRK_Key(BLAS_Fill_Mode(detail::str(j, "uplo")), BLAS_Operation(detail::str(j, "trans")),
                  j["n"].get<int>(), j["k"].get<int>());
}

// {"transA","transC" in "T"/"F"}
inline Json to_json(const SYRK_Options& o) {
  Json j;
  j["transA"] = std::string(o.transpose_A);
  j["transC"] = std::string(o.transpose_C);
  return j;
}
template <>
inline SYRK_Options from_json<SYRK_Options>(const Json& j) {
  return SYRK_Options(Bool_Op(detail::str(j, "transA")), Bool_Op(detail::str(j, "transC")));
}

// SYRK_Options' fields with "transC" in "F"/"T"/"X"
inline Json to_json(const SYRK_Options_Fused& o) {
  Json j;
  j["transA"] = std::string(o.transpose_A);
  j["transC"] = std::string(o.transpose_C);
  return j;
}
template <>
inline SYRK_Options_Fused from_json<SYRK_Options_Fused>(const Json& j) {
  return SYRK_Options_Fused(Bool_Op(detail::str(j, "transA")),
                            Fusable_Bool_Op(detail::str(j, "transC")));
}

// SYRK_Options' fields plus {"tile", "tail"}
inline Json to_json(const SYRK_Options_Tile& o) {
  Json j;
  j["transA"] = std::string(o.transpose_A);
  j["transC"] = std::string(o.transpose_C);
  j["tile"] = std::string(o.tile);
  j["tail"] = std::string(o.tail);
  return j;
}
template <>
inline SYRK_Options_Tile from_json<SYRK_Options_Tile>(const Json& j) {
  return SYRK_Options_Tile(Bool_Op(detail::str(j, "transA")), Bool_Op(detail::str(j, "transC")),
                           Tile_Op(detail::str(j, "tile")), Tail_Op(detail::str(j, "tail")));
}

// {"side" in "Left"/"Right", "uplo", "trans", "diag" in "Unit"/"Non-Unit", "m","n"}
inline Json to_json(const TRSM_Key& key) {
  Json j;
  j["side"] = std::string(key.side);
  j["uplo"] = std::string(key.uplo);
  j["trans"] = std::string(key.trans);
  j["diag"] = std::string(key.diag);
  j["m"] = key.m;
  j["n"] = key.n;
  return j;
}
template <>
inline TRSM_Key from_json<TRSM_Key>(const Json& j) {
  return TRSM_Key(BLAS_Side(detail::str(j, "side")), BLAS_Fill_Mode(detail::str(j, "uplo")),
                  BLAS_Operation(detail::str(j, "trans")), BLAS_Diag(detail::str(j, "diag")),
                  j["m"].get<int>(), j["n"].get<int>());
}

// {"swap_side","transA" in "T"/"F"}
inline Json to_json(const TRSM_Options& o) {
  Json j;
  j["swap_side"] = std::string(o.swap_side);
  j["transA"] = std::string(o.transpose_A);
  return j;
}
template <>
inline TRSM_Options from_json<TRSM_Options>(const Json& j) {
  return TRSM_Options(Bool_Op(detail::str(j, "swap_side")), Bool_Op(detail::str(j, "transA")));
}

// TRSM_Options' fields with "swap_side" in "F"/"T"/"X"
inline Json to_json(const TRSM_Options_Fused& o) {
  Json j;
  j["swap_side"] = std::string(o.swap_side);
  j["transA"] = std::string(o.transpose_A);
  return j;
}
template <>
inline TRSM_Options_Fused from_json<TRSM_Options_Fused>(const Json& j) {
  return TRSM_Options_Fused(Fusable_Bool_Op(detail::str(j, "swap_side")),
                            Bool_Op(detail::str(j, "transA")));
}

// TRSM_Options' fields plus {"tile", "tail", "panel": "auto" | "512" | "1024"}
inline Json to_json(const TRSM_Options_Tile& o) {
  Json j;
  j["swap_side"] = std::string(o.swap_side);
  j["transA"] = std::string(o.transpose_A);
  j["tile"] = std::string(o.tile);
  j["tail"] = std::string(o.tail);
  j["panel"] = std::string(o.panel);
  return j;
}
template <>
inline TRSM_Options_Tile from_json<TRSM_Options_Tile>(const Json& j) {
  return TRSM_Options_Tile(Bool_Op(detail::str(j, "swap_side")), Bool_Op(detail::str(j, "transA")),
                           Tile_Op(detail::str(j, "tile")), Tail_Op(detail::str(j, "tail")),
                           Panel_Op(detail::str(j, "panel")));
}

}  // namespace rtat