// The decode-attention kernels for query groups of 8 heads per KV head.
#define LLMI_GROUP 8
#include "mha_decode_kernels.h"
