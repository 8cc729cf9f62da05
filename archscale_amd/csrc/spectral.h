// Internal interface between the spectral-norm / MuonBall kernels and the C-ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/archscale_muon.h"

namespace archscale {

constexpr int SN_ROWS = 16;         // rows of the Gram matrix per block (4 waves x 4 rows)
constexpr int SN_MAX_CLASSES = 8;   // shape classes per launch (passed by value)

// One shape class of the power iteration inside the workspace.  X is the zero-padded bf16 copy of the matrices with
// the SHORT side first (d_p x L_p), G = X X^T (d_p x d_p), both row-major; d_p is a multiple of 128, L_p of 8.
struct SnClass {
  const __bf16* X;
  const __bf16* G;
  float* z;      // [2][batch][d_p]
  float* part;   // [2][batch][nblk][2]
  float* sigma;  // [batch], result
  int batch, d, d_p, L_p, nblk, tall;
};

struct SnParams {
  int n;
  int blk_start[SN_MAX_CLASSES + 1];  // blocks of class g: batch * nblk
  SnClass c[SN_MAX_CLASSES];
};

// init + `steps` (wide) or `steps + 1` (tall) rounds + final; all classes of one call must be of one kind
hipError_t launch_spectral_iterate(const SnParams& sp, int steps, hipStream_t stream);

hipError_t launch_ball_apply(const muon_ball_item* items, const int32_t* prefix, int n_items, int total_chunks, float lr,
                             float decay, int retract_mode, float retract_step, float* log_out, hipStream_t stream);

}  // namespace archscale
