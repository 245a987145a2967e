// The decode-attention kernels for query groups of 4 heads per KV head.
#define LLMI_GROUP 4
#include "mha_decode_kernels.h"
