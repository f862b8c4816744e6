// Kernel parameter blocks of the zoo state / output kernels, shared by the rotated-storage kernels and the
// canonical-storage (in-kernel un-rotation) variants.
#pragma once

#include "zoo_common.h"

struct ZooStateParams {
  const int8_t* kqT;
  const int8_t* vqT;
  const int8_t* wq;
  const _Float16* u;
  const float* fw;
  const float* ev;
  const float* gam;
  const float* pack;  // fw | ev | gam per (batch, chunk, head), 64 + 64 + K floats, or nullptr
  int8_t* h_i8;
  _Float16* e_out;
  float* ht;
  const float* skw;
  const float* svw;
  const float* sw;
  const float* ss;
  const _Float16* unrot;
  int qmax;
  int bf;  // activations are bf16
  int T, H, V, NT;
  int S;  // 64-token pieces per chunk (1; 2..4 in the kernels' PAIR mode)
};

struct ZooOutParams {
  const _Float16* q;
  const _Float16* k;
  const _Float16* v;
  const int8_t* h_i8;
  const float* g;
  const _Float16* A;
  const int8_t* qg;
  const int8_t* qc;  // ready-made local codes of q, k (B,T,H,K) and v (B,T,H,V): q, k, v are then not read
  const int8_t* kc;
  const int8_t* vc;
  void* o;
  int o_is_f32;
  const float* sq;
  const float* sk;
  const float* svl;
  const float* ss;
  const _Float16* unrot;
  float scale;
  int qmax;
  int bf;  // activations (and a 16-bit output) are bf16
  int B, T, H, V, NT;
  const _Float16* Ax;  // 128-token chunks under per-channel decay: (B,T,H,64) fp16 from the cross launch of the A kernel
  float* cross;  // chunks of S > 1 pieces: fp32 (B,T,H,V) partial local products of the later pieces, else nullptr
  int S;         // 64-token pieces per chunk (and per stored state): 1, or 2..4
  int cross_j;   // cross launch j = 1 .. S-1: piece s >= j of a chunk takes its product with the tokens of piece j - 1
};

// 128-token chunks under per-channel decay: the second halves' blocks of the intra-chunk product with the first halves' tokens
struct ZooACrossParams {
  const _Float16* q;
  const _Float16* k;
  const float* g;
  _Float16* Ax;  // (B,T,H,64) fp16, rows of the second halves
  const float* sq;
  const float* sk;
  const _Float16* rot;
  const float* dq;
  float scale;
  int qmax;
  int bf;
  int B, T, H;
};
int zoo_gla_A_cross_launch(const ZooACrossParams& p, int K, hipStream_t stream);  // defined in zoo_gla_A_cross.hip

// canonical storage: one workgroup spans all V value channels (V = 64 or 128); defined in zoo_unrot.hip
int zoo_state_unrot_launch(const ZooStateParams& p, bool delta, int K, int batch, bool pair, hipStream_t stream);
int zoo_output_unrot_launch(const ZooOutParams& p, int decay, int K, hipStream_t stream);
