#include "fattn_common.h"
bool fattn_mma_supported(const FattnArgs &, int) { return false; }
int fattn_mma_launch(const FattnArgs &, int, hipStream_t) { return (int)hipErrorNotSupported; }
