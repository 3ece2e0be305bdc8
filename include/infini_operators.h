/* Source-compatible umbrella: callers of the reference include this name
 * (reference include/infini_operators.h:1-19), which pulls one header per
 * operator.  The operators this library does not implement (the CNN family:
 * avg_pool, conv, expand, gemm, global_avg_pool, max_pool, relu) have no
 * header here. */
#include "handle/handle_export.h"
#include "ops/add/add.h"
#include "ops/add_rms_norm/add_rms_norm.h"
#include "ops/attention/attention.h"
#include "ops/causal_softmax/causal_softmax.h"
#include "ops/matmul/matmul.h"
#include "ops/mlp/mlp.h"
#include "ops/random_sample/random_sample.h"
#include "ops/rearrange/rearrange.h"
#include "ops/rms_norm/rms_norm.h"
#include "ops/rotary_embedding/rotary_embedding.h"
#include "ops/swiglu/swiglu.h"
#include "tensor/tensor_descriptor.h"
