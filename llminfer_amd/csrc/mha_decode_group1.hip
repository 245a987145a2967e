// The decode-attention kernels for query groups of one head per KV head.
#define LLMI_GROUP 1
#include "mha_decode_kernels.h"
