// The decode-attention kernels for query groups of 2 heads per KV head.
#define LLMI_GROUP 2
#include "mha_decode_kernels.h"
