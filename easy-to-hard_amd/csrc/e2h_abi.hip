// Library identity, status strings and the option store of libe2h_quant.so.
#include <string.h>

#include "e2h_common.h"

namespace e2h {
Options &options() {
  static Options o = {};
  return o;
}
}  // namespace e2h

extern "C" int e2h_abi_version(void) { return E2H_ABI_VERSION; }

extern "C" const char *e2h_status_string(int status) {
  switch (status) {
    case E2H_OK: return "ok";
    case E2H_ERR_NULL_POINTER: return "a required pointer is NULL";
    case E2H_ERR_BAD_SHAPE: return "unsupported shape (m, n, k)";
    case E2H_ERR_BAD_GROUPSIZE: return "groupsize must be one of 32, 64, 128, 256 and divide k";
    case E2H_ERR_BAD_INNER_K_TILES: return "inner_k_tiles must be one of 2, 4, 8 and 16*inner_k_tiles must divide k";
    case E2H_ERR_MISALIGNED: return "pointer not aligned as required";
    case E2H_ERR_LAUNCH: return "HIP kernel launch failed";
    case E2H_ERR_NO_DEVICE: return "no gfx950 device";
    case E2H_ERR_BAD_OPTION: return "unknown option or value out of range";
    case E2H_ERR_SCRATCH_TOO_SMALL: return "the call needs more scratch memory than the library's fixed buffer holds";
    default: return "unknown status";
  }
}

extern "C" int e2h_set_option(const char *name, int value) {
  if (!name) return E2H_ERR_NULL_POINTER;
  e2h::Options &o = e2h::options();
  if (!strcmp(name, "int4_rows_per_wave") || !strcmp(name, "int8_rows_per_wave")) {
    if (value != 0 && value != 16 && value != 32 && value != 64) return E2H_ERR_BAD_OPTION;
    (name[3] == '4' ? o.int4_rows_per_wave : o.int8_rows_per_wave) = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_k_slices")) {
    if (value < 0 || value > 16) return E2H_ERR_BAD_OPTION;
    o.int4_k_slices = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_k_groups")) {
    if (value != 0 && value != 1 && value != 2 && value != 4) return E2H_ERR_BAD_OPTION;
    o.int4_k_groups = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_col_waves")) {
    if (value < 0 || value > 4) return E2H_ERR_BAD_OPTION;
    o.int4_col_waves = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_k_groups")) {
    if (value < 0 || value > 2) return E2H_ERR_BAD_OPTION;
    o.int8_k_groups = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_force_generic")) {
    o.int8_force_generic = value != 0;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_k_slices")) {
    if (value < 0 || value > 16) return E2H_ERR_BAD_OPTION;
    o.int8_k_slices = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_no_xsum")) {
    o.int4_no_xsum = value != 0;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_no_gemm32")) {
    o.int4_no_gemm32 = value != 0;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_gemm32_min_rows")) {
    if (value < 0) return E2H_ERR_BAD_OPTION;
    o.int4_gemm32_min_rows = value;
    return E2H_OK;
  }
  if (!strcmp(name, "row_tiles")) {
    if (value != 0 && value != 1 && value != 2 && value != 4) return E2H_ERR_BAD_OPTION;
    o.row_tiles = value;
    return E2H_OK;
  }
  if (!strcmp(name, "attention_waves")) {
    if (value != 0 && value != 4 && value != 8) return E2H_ERR_BAD_OPTION;
    o.attention_waves = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_gemm_waves")) {
    if (value != 0 && value != 4 && value != 8) return E2H_ERR_BAD_OPTION;
    o.int8_gemm_waves = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_gemm_wave_cols")) {
    if (value != 0 && value != 2 && value != 4) return E2H_ERR_BAD_OPTION;
    o.int8_gemm_wave_cols = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int4_gemm_tile")) {
    if (value != 0 && value != 128 && value != 256) return E2H_ERR_BAD_OPTION;
    o.int4_gemm_tile = value;
    return E2H_OK;
  }
  if (!strcmp(name, "int8_gemm_tile")) {
    if (value != 0 && value != 128 && value != 256) return E2H_ERR_BAD_OPTION;
    o.int8_gemm_tile = value;
    return E2H_OK;
  }
  if (!strcmp(name, "staged_tiles") || !strcmp(name, "staged_slices")) {
    if (value < 0 || value > 16) return E2H_ERR_BAD_OPTION;
    (name[7] == 't' ? o.staged_tiles : o.staged_slices) = value;
    return E2H_OK;
  }
  if (!strcmp(name, "staged_no_rows64")) {
    o.staged_no_rows64 = value != 0;
    return E2H_OK;
  }
  if (!strcmp(name, "attention_no_mfma")) {
    o.attention_no_mfma = value != 0;
    return E2H_OK;
  }
  return E2H_ERR_BAD_OPTION;
}
