// The one-token quantized linear for 4-bit weights (see token_linear_impl.h).
#define OQ_TOKEN_LINEAR_BITS 4
#include "token_linear_impl.h"
