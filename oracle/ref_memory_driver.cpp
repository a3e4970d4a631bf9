// TEST INFRASTRUCTURE -- not part of the product.
//
// C entry point over the reference's own memory planner, compiled from the
// sources where they lie under /root/reference (src/structure/memory/
// {greedy,linear,info,index}.cpp) by oracle/Makefile into
// oracle/_ref/libref_memory.so.  Tests use it to check both the product's
// planner and the Python restatement in oracle/memory_plan.py, offset for
// offset, on seeded lifetime sets.
#include <cstddef>
#include <cstdint>
#include <memory>
#include <string>

#include "structure/memory/greedy.h"
#include "structure/memory/index.h"
#include "structure/memory/info.h"
#include "structure/memory/linear.h"

// kind 0 = PlainInfos + LinearPlan, 1 = GreedyInfos + GreedyPlan (the pairs
// reference src/worker/planner.cpp:322-340 builds).  Tensors are pushed in
// array order under the names "t0", "t1", ...; offsets[i] receives
// Index::Get("t<i>") and *maximum receives Index::GetMaximum().
extern "C" int ref_memory_plan(int kind, int n, const uint64_t *starts, const uint64_t *ends, const uint64_t *sizes,
                               uint64_t *offsets, uint64_t *maximum) {
  using namespace fluidml::memory;
  std::unique_ptr<Infos> infos;
  std::unique_ptr<Plan> plan;
  if (kind == 0) {
    infos = std::make_unique<PlainInfos>();
    plan = std::make_unique<LinearPlan>();
  } else if (kind == 1) {
    infos = std::make_unique<GreedyInfos>();
    plan = std::make_unique<GreedyPlan>();
  } else {
    return -1;
  }
  for (int i = 0; i < n; ++i) {
    infos->Push(Info("t" + std::to_string(i), starts[i], ends[i], sizes[i]));
  }
  Index index = plan->Run(*infos);
  for (int i = 0; i < n; ++i) offsets[i] = index.Get("t" + std::to_string(i));
  *maximum = index.GetMaximum();
  return 0;
}
