// The one-token quantized linear for 2-bit weights (see token_linear_impl.h).
#define OQ_TOKEN_LINEAR_BITS 2
#include "token_linear_impl.h"
