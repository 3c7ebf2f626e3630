// Harness in the shape of the reference's sample nccl-overlap/samples/multi-process-adam-scattered.cpp, for one GPU:
// one gradient / weight buffer per "parent buffer", moments in single arrays, the sample's integer input pattern
// ((i%2+1)*(index%20+1) for buffer i, :221-226), beta1 = beta2 = .5, alpha = 1, epsilon 1e-6, five checked epochs
// (:320, :345).  Where the sample calls ncclAllReduceScatteredAdam / ncclAllReduceScatteredLAMB this calls
// ccn_adam_f32_scattered / ccn_lamb_f32_scattered over P resident rank buffers, and where it calls
// check_epoch_results_adam / check_epoch_results_lamb (:81-153, :371-462) this runs the CPU oracle and the sample's
// comparator (eq_float, :60-66) on every element.
//
//   adam_lamb_scattered <adam|lamb> [ranks=2] [scale_down=16] [max_buff_size=0]
// Buffer sizes: head and tail of the sample's list (:736), the large ones divided by scale_down to fit a test.
// max_buff_size > 0 (lamb): every parent buffer is cut into small buffers of at most that many elements, each an
// allocation of its own, with the sample's smallBufferIdToParentBufferId map (:505-517); the norms stay per parent.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "ccn_oracle.h"
#include "coconet_hip.h"

#define CCNCHECK(cmd)                                                                                   \
  do {                                                                                                  \
    int rc_ = (cmd);                                                                                    \
    if (rc_ != CCN_OK) {                                                                                \
      printf("Failed, coconet_hip error %s:%d '%s'\n", __FILE__, __LINE__, ccn_strerror(rc_));          \
      exit(EXIT_FAILURE);                                                                               \
    }                                                                                                   \
  } while (0)

int main(int argc, char** argv) {
  if (argc < 2) {
    printf("usage: %s <adam|lamb> [ranks=2] [scale_down=16] [max_buff_size=0]\n", argv[0]);
    return 1;
  }
  const bool lamb = std::string(argv[1]) == "lamb";
  const int P = argc > 2 ? atoi(argv[2]) : 2;
  const size_t down = argc > 3 ? (size_t)atoi(argv[3]) : 16;
  const size_t listed[] = {31260672, 2048, 1048576, 1048576, 1048576, 1048576, 4194304, 4194304,
                           1024,     1024, 1024,    1024,    30528,   1024,    1024,    1024};
  const size_t max_buff = argc > 4 ? (size_t)atoll(argv[4]) : 0;
  std::vector<size_t> parent_sizes;
  for (size_t s : listed) parent_sizes.push_back(s > (1u << 20) ? s / down : s);
  const int nparents = (int)parent_sizes.size();
  std::vector<size_t> parent_offs(nparents + 1, 0);
  for (int i = 0; i < nparents; i++) parent_offs[i + 1] = parent_offs[i] + parent_sizes[i];
  // the buffers the calls see: the parents themselves, or their pieces
  std::vector<size_t> sizes, parent_of;
  for (int i = 0; i < nparents; i++) {
    if (lamb && max_buff > 0) {
      for (size_t lo = 0; lo < parent_sizes[i]; lo += max_buff) {
        sizes.push_back(parent_sizes[i] - lo < max_buff ? parent_sizes[i] - lo : max_buff);
        parent_of.push_back((size_t)i);
      }
    } else {
      sizes.push_back(parent_sizes[i]);
      parent_of.push_back((size_t)i);
    }
  }
  const int nbuffs = (int)sizes.size();
  std::vector<size_t> offs(nbuffs + 1, 0);
  for (int i = 0; i < nbuffs; i++) offs[i + 1] = offs[i] + sizes[i];
  const size_t total = offs[nbuffs];

  CCNCHECK(ccn_init(0));
  // host copies (the checker's state) and device buffers
  std::vector<float> hg(total), hw(total), hm(total, 0.f), hv(total, 0.f);
  for (int i = 0; i < nparents; i++)
    for (size_t index = 0; index < parent_sizes[i]; index++)
      hg[parent_offs[i] + index] = hw[parent_offs[i] + index] = (float)(i % 2 + 1) * (float)(index % 20 + 1);
  std::vector<const float*> g_ptrs((size_t)P * nbuffs);
  std::vector<float*> w_ptrs(nbuffs);
  for (int p = 0; p < P; p++)
    for (int i = 0; i < nbuffs; i++) {
      float* d;
      CCNCHECK(ccn_malloc((void**)&d, sizes[i] * sizeof(float)));
      CCNCHECK(ccn_memcpy_h2d(d, hg.data() + offs[i], sizes[i] * sizeof(float), nullptr));
      g_ptrs[(size_t)p * nbuffs + i] = d;
    }
  for (int i = 0; i < nbuffs; i++) {
    CCNCHECK(ccn_malloc((void**)&w_ptrs[i], sizes[i] * sizeof(float)));
    CCNCHECK(ccn_memcpy_h2d(w_ptrs[i], hw.data() + offs[i], sizes[i] * sizeof(float), nullptr));
  }
  float *m, *v;
  CCNCHECK(ccn_malloc((void**)&m, total * sizeof(float)));
  CCNCHECK(ccn_malloc((void**)&v, total * sizeof(float)));
  CCNCHECK(ccn_fill_f32(m, 0.f, total, nullptr));
  CCNCHECK(ccn_fill_f32(v, 0.f, total, nullptr));
  CCNCHECK(ccn_stream_sync(nullptr));

  const float alpha = 1.0f, beta1 = 0.5f, beta2 = 0.5f, eps = 1e-6f;
  ccn_scatter_plan* sp = nullptr;
  ccn_lamb_plan* lp = nullptr;
  if (lamb && max_buff > 0) CCNCHECK(ccn_lamb_plan_create_parented(sizes.data(), parent_of.data(), nbuffs, &lp));
  else if (lamb) CCNCHECK(ccn_lamb_plan_create(offs.data(), nbuffs, &lp));
  else CCNCHECK(ccn_scatter_plan_create(sizes.data(), nbuffs, &sp));

  std::vector<const float*> og(P, hg.data());   // every rank holds the same gradients, as in the sample
  std::vector<float> got(total);
  bool ok = true;
  for (int iter = 0; iter < 5 && ok; iter++) {
    // the sample's stepsize is +alpha; this library takes the learning rate, lr = -alpha
    if (lamb)
      CCNCHECK(ccn_lamb_f32_scattered(lp, g_ptrs.data(), P, w_ptrs.data(), m, v, -alpha, beta1, beta2, eps, 1.0f, iter + 1,
                                      CCN_LAMB_REFERENCE, nullptr));
    else
      CCNCHECK(ccn_adam_f32_scattered(sp, g_ptrs.data(), P, w_ptrs.data(), m, v, -alpha, beta1, beta2, eps, iter + 1, nullptr));
    for (int i = 0; i < nbuffs; i++)
      CCNCHECK(ccn_memcpy_d2h(got.data() + offs[i], w_ptrs[i], sizes[i] * sizeof(float), nullptr));
    CCNCHECK(ccn_stream_sync(nullptr));
    if (lamb) orc_lamb_f32(og.data(), P, hw.data(), hm.data(), hv.data(), parent_offs.data(), nparents, -alpha, beta1, beta2, eps,
                           1.0f, iter + 1, 1, nullptr);
    else orc_adam_f32(og.data(), P, hw.data(), hm.data(), hv.data(), total, -alpha, beta1, beta2, eps, iter + 1);
    for (size_t i = 0; i < total; i++) {
      if (!orc_eq_float_1e5(hw[i], got[i])) {
        printf("Mismatch at epoch %d, element %zu: ref '%.9g', computed '%.9g'\n", iter, i, hw[i], got[i]);
        ok = false;
        break;
      }
    }
    if (ok) printf("Epoch %d: %s weights match the checker on %zu elements in %d buffers of %d parents\n", iter, lamb ? "LAMB" : "Adam", total, nbuffs, nparents);
  }
  if (lamb) CCNCHECK(ccn_lamb_plan_destroy(lp));
  else CCNCHECK(ccn_scatter_plan_destroy(sp));
  for (auto p : g_ptrs) CCNCHECK(ccn_free((void*)p));
  for (auto p : w_ptrs) CCNCHECK(ccn_free(p));
  CCNCHECK(ccn_free(m));
  CCNCHECK(ccn_free(v));
  printf(ok ? "Success\n" : "Failure\n");
  return ok ? 0 : 2;
}
