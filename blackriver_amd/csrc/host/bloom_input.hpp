// Batch preparation for the BLOOM block: what the reference's rank-0 feeder
// computes per batch (BloomInput::fetch_data, blackriver/train_bloom.cpp:41-93).
// Host versions work on plain buffers; the device versions are exposed as the
// words bloom.embed / bloom.alibi / bloom.xmask and fill device tensors
// directly instead of shipping the tables across PCIe.
#pragma once

#include <cstdint>
#include <vector>

#include "vm.hpp"

namespace br {

struct BloomInput {
    // xinput[i,:] = vocab[ids[i],:]
    static void gather_embeddings(const float* vocab, int64_t hidden, const int32_t* ids, int64_t n, float* xinput);
    // alibi[h,k] = (float)(k * slope_h), slope_h = (2^(-2^(3-log2(heads))))^(h+1) in fp64
    static void build_alibi(int64_t heads, int64_t tokens, float* alibi);
    // xmask[b,q,k] = 0 when k <= q and mask[b,0..k] are all non-zero, else -FLT_MAX
    static void build_xmask(const int32_t* mask, int64_t batch, int64_t tokens, float* xmask);
};

// Registers bloom.embed ( ids_cpu_int table_dev out_dev -- ),
// bloom.alibi ( alibi_dev -- ) and bloom.xmask ( mask_cpu_int xmask_dev -- ).
void load_bloom_words(Enviroment& env);

}  // namespace br
