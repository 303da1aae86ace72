// Differential attention for prompt portions on the matrix cores (bf16).
#include "attention_diff.h"

namespace ninfer {

bool diff_attention_tiles_takes(const DiffAttnArgs& a) { return false; }
int diff_attention_tiles(const DiffAttnArgs& a, hipStream_t stream) {
  return set_error(-1, "diff_attention: no tile kernel for this shape");
}

}  // namespace ninfer
