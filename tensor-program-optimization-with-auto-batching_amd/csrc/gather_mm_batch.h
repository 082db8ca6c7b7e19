// What the batched gather-matmul entry point and its two-pass streaming kernels share.
#pragma once
#include "lora_device.h"

// One problem of a batch: device pointers laid out as mlora_gather_mm takes them.
struct GmmSet {
  void* y;
  const f16* x;
  const f16* A;
  const f16* B;
};

// shrink pass + expand pass over n_sets problems; ws holds n_sets * kc * T * r floats.  Arguments are validated by the caller.
int gmm_batch_stream(const GmmSet* sets, int n_sets, int y_dtype, int ldy, int x_layout, const int32_t* ids, float scaling,
                     int T, int K, int N, int r, int n_ad, float* ws, hipStream_t s);
