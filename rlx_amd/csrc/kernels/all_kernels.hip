// Single translation unit for the gfx950 code object the host library embeds and loads with hipModuleLoadData.
#include "dequant.hip"
#include "fakequant.hip"
#include "gemm.hip"
#include "gemv.hip"
#include "moe.hip"
#include "rowops.hip"
#include "topk.hip"
