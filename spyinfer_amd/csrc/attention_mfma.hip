#include "common.h"
extern "C" int64_t spy_attention_mfma_workspace(int num_tiles, int n_kv, int d, int splits) { return 0; }
extern "C" int spy_attention_mfma() { return spy_fail("spy_attention_mfma: not built yet"); }
