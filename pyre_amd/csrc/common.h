// Internal definitions shared by the translation units of libpyre_hip.so (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>
#include <string>
#include <vector>
#include "../../include/pyre_hip.h"

#define PYRE_WAVE 64
#define PYRE_UNIT 64            // weights per decode unit (one lane decodes one unit at a time)

struct pyre_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  std::string err;
  // split-K workspace: partial sums [ksplit][t][rows64] and one self-resetting ticket counter per row tile
  float* ws_partial = nullptr; size_t ws_partial_bytes = 0;
  uint32_t* ws_ticket = nullptr; size_t ws_ticket_n = 0;
  // staging for host-pointer entry points
  void* stage = nullptr; size_t stage_bytes = 0;
  // expanded codebooks in device memory: iq3s u32[512], iq2xs u64[512]
  uint32_t* d_iq3s = nullptr; uint64_t* d_iq2xs = nullptr;
};

extern thread_local std::string g_pyre_create_err;

int pyre_fail(pyre_ctx* ctx, int code, const char* fmt, ...);
#define PYRE_HIP(ctx, call) do { hipError_t e_ = (call); if (e_ != hipSuccess) return pyre_fail((ctx), PYRE_E_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__, __LINE__); } while (0)
#define PYRE_CHECK_LAUNCH(ctx) PYRE_HIP(ctx, hipGetLastError())

int pyre_stage(pyre_ctx* ctx, size_t nbytes, void** out);          // grow-only device staging buffer
int pyre_workspace(pyre_ctx* ctx, size_t partial_bytes, size_t tickets);

// ---- device-side matrix view --------------------------------------------------------------------------------------
// Weights live in "lane = row" planes: rows are grouped in tiles of 64, and for every (tile, unit) the 64 rows'
// entries of a plane are contiguous, so one wave (lane l = row l of the tile) reads every plane with fully
// coalesced loads while all lanes sit on the same 64 columns (activations then come from scalar loads).
//   vector plane  p0: [tile][unit][chunk < V][lane] x 16 B
//   small planes  p1..p3: [tile][unit][lane] x e bytes
//   block plane   pb: [tile][unit/4][lane] x e bytes    (per 256-value super-block)
struct QMatDev {
  const uint8_t* p0; const uint8_t* p1; const uint8_t* p2; const uint8_t* p3; const uint8_t* pb;
  int rows, cols, U, tiles, fmt;
};

struct pyre_qmat {
  pyre_ctx* ctx; uint32_t ty; size_t rows, cols; size_t gguf_bytes;
  void* base; size_t dev_bytes; QMatDev dv;
};

// launchers implemented in qmat.hip, used by the block / model code
int pyre_gemv_launch(pyre_ctx* ctx, const QMatDev& m, const float* x_dev, int t, float* y_dev);
int pyre_row_launch(pyre_ctx* ctx, const QMatDev& m, const uint32_t* row_idx_dev, int n, float* out_dev, int out_stride);
