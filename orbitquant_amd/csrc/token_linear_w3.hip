// The one-token quantized linear for 3-bit weights (see token_linear_impl.h).
#define OQ_TOKEN_LINEAR_BITS 3
#include "token_linear_impl.h"
