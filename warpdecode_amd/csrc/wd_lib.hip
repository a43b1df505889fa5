// Single translation unit of libwarpdecode_amd.so.
#include "wd_ops.hip"
#include "wd_layer.hip"
#include "wd_noalloc.hip"
#include "wd_cache.hip"
#include "wd_stack.hip"
#include "wd_gguf.hip"
