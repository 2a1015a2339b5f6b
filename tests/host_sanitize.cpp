// Exercises the host-only half of the launchers (torch_mlu_amd/csrc/fa_host.h: validation, kernel choice, workspace
// sizes) over a grid of ordinary, extreme and malformed parameter blocks.  Built by tests/test_cabi_host.py with
// -fsanitize=address,undefined -fno-sanitize-recover: any overflow, out-of-bounds access or other undefined behaviour
// aborts the run.  Prints the number of blocks it pushed through.
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <initializer_list>

#include "fa_host.h"

using namespace fa::host;

// a * b * c, capped (the driver itself must not overflow while it builds strides for absurd sizes)
static int64_t mul3(int64_t a, int64_t b, int64_t c) {
  const __int128 v = (__int128)a * b * c;
  return v > ((__int128)1 << 60) ? ((int64_t)1 << 60) : (int64_t)v;
}

static fa_fwd_params good_fwd(int B, int Hq, int Hk, int Sq, int Sk, int D) {
  fa_fwd_params p;
  memset(&p, 0, sizeof(p));
  p.q = (void*)0x1000; p.k = (void*)0x2000; p.v = (void*)0x3000; p.out = (void*)0x4000; p.lse = (float*)0x5000;
  p.q_stride_b = mul3(Sq, Hq, D); p.q_stride_s = mul3(Hq, D, 1); p.q_stride_h = D;
  p.k_stride_b = mul3(Sk, Hk, D); p.k_stride_s = mul3(Hk, D, 1); p.k_stride_h = D;
  p.v_stride_b = p.k_stride_b; p.v_stride_s = p.k_stride_s; p.v_stride_h = D;
  p.o_stride_b = p.q_stride_b; p.o_stride_s = p.q_stride_s; p.o_stride_h = D;
  p.lse_stride_b = mul3(Hq, Sq, 1); p.lse_stride_h = Sq; p.lse_stride_s = 1;
  p.batch = B; p.heads_q = Hq; p.heads_k = Hk; p.seqlen_q = Sq; p.seqlen_k = Sk; p.head_dim = D;
  p.scale = 0.088f; p.dtype = FA_DTYPE_BF16;
  return p;
}

static long push_fwd(const fa_fwd_params& p) {
  long n = 0;
  const int rc = validate(&p);
  if (rc == FA_OK) {
    int k = -1, s = -1;
    plan(&p, &k, &s);
    const size_t ws = workspace_bytes(&p, k, s);
    n += (long)(ws & 1) + k + s;  // keep the results alive
  }
  return n + 1000003;
}

int main() {
  long sink = 0, count = 0;
  const int32_t big = 0x7fffffff;
  for (int B : {1, 2, 64, 4096, big})
    for (int Hq : {1, 8, 32, 128, big})
      for (int Hk : {1, 2, 8})
        for (int Sq : {0, 1, 2, 4, 16, 17, 127, 128, 129, 256, 4096, 131072, big})
          for (int Sk : {0, 1, 255, 256, 8192, 131072, big})
            for (int D : {8, 64, 72, 128, 256}) {
              fa_fwd_params p = good_fwd(B, Hq, Hk, Sq, Sk, D);
              for (int causal : {0, 1, 2})
                for (int kern : {0, 1, 2, 3, 4, 5})
                  for (int ns : {0, 1, 7, 64}) {
                    p.is_causal = causal; p.kernel = kern; p.num_splits = ns;
                    sink += push_fwd(p); ++count;
                  }
              p.kernel = 0; p.num_splits = 0; p.is_causal = 1;
              p.dropout_p = 0.3f; sink += push_fwd(p); ++count;
              p.dropout_p = 0.f; p.bias = (void*)0x8000; p.bias_stride_q = Sk & ~3; sink += push_fwd(p); ++count;
              p.bias = nullptr;
              p.cu_seqlens_q = (const int32_t*)0x6000; p.cu_seqlens_k = (const int32_t*)0x7000; sink += push_fwd(p); ++count;
            }
  // malformed blocks: extreme strides, negative sizes, odd alignments
  for (int64_t st : std::initializer_list<int64_t>{-8, 0, 7, (int64_t)1 << 24, (int64_t)1 << 40, (int64_t)(INT64_MAX & ~(int64_t)7), INT64_MIN}) {
    fa_fwd_params p = good_fwd(2, 8, 2, 128, 256, 128);
    p.q_stride_s = st; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.k_stride_s = st; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.o_stride_b = st; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.lse_stride_h = st; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.bias = (void*)0x8000; p.bias_stride_b = st; sink += push_fwd(p); ++count;
  }
  for (int v : {-1, 0, -big - 1}) {
    fa_fwd_params p = good_fwd(2, 8, 2, 128, 256, 128);
    p.batch = v; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.heads_k = v; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.seqlen_q = v; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.head_dim = v; sink += push_fwd(p); ++count;
    p = good_fwd(2, 8, 2, 128, 256, 128); p.kernel = v; sink += push_fwd(p); ++count;
  }
  sink += validate(nullptr);
  // backward
  for (int B : {1, 64, big})
    for (int Hq : {1, 32, big})
      for (int Sq : {0, 1, 4096, big})
        for (int D : {8, 128, 256, 264})
          for (int packed : {0, 1}) {
            fa_bwd_params p;
            memset(&p, 0, sizeof(p));
            p.q = p.k = p.v = p.out = p.dout = (void*)0x1000; p.lse = (const float*)0x2000;
            p.dq = p.dk = p.dv = (void*)0x3000;
            if (packed) { p.cu_seqlens_q = p.cu_seqlens_k = (const int32_t*)0x4000; p.total_q = mul3(B, Sq, 1); }
            p.q_stride_s = p.k_stride_s = p.v_stride_s = p.o_stride_s = p.do_stride_s = p.dq_stride_s = p.dk_stride_s =
                p.dv_stride_s = mul3(Hq, D, 1);
            p.q_stride_h = p.k_stride_h = p.v_stride_h = p.o_stride_h = p.do_stride_h = p.dq_stride_h = p.dk_stride_h =
                p.dv_stride_h = D;
            p.lse_stride_h = Sq; p.lse_stride_s = 1;
            p.batch = B; p.heads_q = Hq; p.heads_k = Hq; p.seqlen_q = Sq; p.seqlen_k = Sq; p.head_dim = D;
            p.scale = 0.1f; p.dtype = FA_DTYPE_FP16; p.is_causal = 1;
            if (bwd_validate(&p) == FA_OK) sink += (long)(bwd_ws_bytes(&p) & 3);
            ++count;
          }
  sink += bwd_validate(nullptr);
  printf("%ld blocks (%ld)\n", count, sink);
  return 0;
}
