// Kernel argument block shared by the host launchers and the device kernels.
#pragma once
#include <stdint.h>

namespace moda {

struct Str3 {
  int64_t b, t, h;
};

struct KArgs {
  const uint16_t *q, *k, *v, *kd, *vd, *o, *d_o;
  uint16_t *out_o, *dq, *dk, *dv, *dkd, *dvd;
  float* lse;          // [B, Tq, Hq]   (written by forward, read by backward)
  float* delta;        // [B, Hq, Tq]   workspace: MINUS rowsum(o * do)
  Str3 sq, sk, sv, skd, svd, so, sdo, sdq, sdk, sdv, sdkd, sdvd;
  int B, T, Hkv;
  int Tq;    // query rows per (batch, query head)
  int Gf;    // query rows per token (fold factor)
  int Hq;    // query-head programs per batch
  int hdiv;  // kv head = hq / hdiv
  int L;     // depth slots per token in the depth tensors (row t*L + l = slot l of token t)
  int Lv;    // slots per token that hold data, 1 <= Lv <= L: slots l >= Lv are invisible
  int Cb;    // chunk-visible: tokens per chunk
  int has_seq, causal, chunk;
  int nqt;   // query tiles per (batch, query head)
  float scale;
  int compute_units;  // of the device the launch goes to (host-side launch-shape decisions)
};

}  // namespace moda
