// The decode-attention kernels for query groups of 16 heads per KV head.
#define LLMI_GROUP 16
#include "mha_decode_kernels.h"
