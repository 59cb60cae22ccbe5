// Layout of the stored dS of the RetNet backward (written by the row pass of bwd_chain.h, read by dk_from_ds.h):
// 64 x 64 blocks of 8 KB, [B*H][S_q/64][S_kv/64][64][64] fp16.
#pragma once
#include <cstddef>

#include "../../utils/cdna4.h"

namespace aat {

// Offset (in elements) of dS[bh][q][kv].
AAT_DEV size_t ds_block_offset(int bh, int q, int kv, int seq_q, int seq_k) {
  return ((((size_t)bh * (seq_q >> 6) + (q >> 6)) * (seq_k >> 6) + (kv >> 6)) << 12) + ((q & 63) << 6) + (kv & 63);
}

}  // namespace aat
