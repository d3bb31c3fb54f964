// Uses the installed headers and both libraries without touching a GPU: a closure and a
// shard of the host layer, the dispatch table's HIP column, and a pure-host C-ABI call.
#include <cstdio>
#include <cstring>

#include "hip_ops.h"
#include "minerva_types.h"
#include "mnv_hip.h"
#include "op_dispatch.h"

int main() {
  minerva::ArithmeticClosure closure{minerva::ArithmeticType::kAdd};
  minerva::Scale extent{3, 4};
  minerva::DataShard shard(nullptr, extent);
  if (shard.size_.Prod() != 12) return 1;
  minerva::ArithmeticOp op;
  op.closure = closure;
  if (op.Name() != "+") return 2;
  if (std::strcmp(mnv_error_string(0), "ok") != 0) return 3;
  if (mnv_pooled_size(55, 3, 2, 0) != 27) return 4;
  std::printf("consumer OK\n");
  return 0;
}
