// Arena planning: which byte offset every intermediate tensor and every node
// scratch buffer gets inside the one HBM arena.  Offsets must equal FluidML's
// own plan bit for bit, so the two planners restate the reference's decision
// procedure (src/structure/memory/{info,index,linear,greedy}.cpp) including
// the places where it is not what a textbook best-fit would do; each such
// place is called out below.
#ifndef FLUIDML_AMD_HOST_STRUCTURE_MEMORY_MEMORY_H_
#define FLUIDML_AMD_HOST_STRUCTURE_MEMORY_MEMORY_H_

#include <cstddef>
#include <list>
#include <queue>
#include <string>
#include <tuple>
#include <unordered_map>
#include <vector>

namespace fluidml {
namespace memory {

// One request: `size` bytes alive over node indices [start, end] (reference info.h:11-31).
class Info {
 public:
  Info(std::string &&name, size_t start, size_t end, size_t size);
  const std::string &GetName() const;
  size_t GetStart() const;
  size_t GetEnd() const;
  size_t GetSize() const;

 private:
  std::string name_;
  size_t start_, end_, size_;
};

// Queue of requests; the order it pops in is the placement order (info.h:33-71).
class Infos {
 public:
  virtual ~Infos() = default;
  virtual bool IsEmpty() const = 0;
  virtual void Push(Info &&info) = 0;
  virtual Info Pop() = 0;
};

// FIFO (info.cpp:23-34).
class PlainInfos : public Infos {
 public:
  bool IsEmpty() const override;
  void Push(Info &&info) override;
  Info Pop() override;

 private:
  std::list<Info> infos_;
};

// Largest request first.  The comparator looks at the size only, so the order
// among equal sizes is whatever std::priority_queue's binary heap yields for
// the push sequence (info.cpp:36-52); BERT has dozens of equal-sized tensors,
// hence the same container is used here.
class GreedyInfos : public Infos {
 public:
  struct InfoCompare {
    bool operator()(const Info &lhs, const Info &rhs) const;
  };
  bool IsEmpty() const override;
  void Push(Info &&info) override;
  Info Pop() override;

 private:
  std::priority_queue<Info, std::vector<Info>, InfoCompare> infos_;
};

// name -> (offset, size) (index.h:11-25, index.cpp:8-28). Set keeps the first
// value given for a name.
class Index {
 public:
  size_t Get(const std::string &name) const;  // throws std::out_of_range for an unknown name
  bool Has(const std::string &name) const;
  size_t GetSize(const std::string &name) const;
  size_t GetMaximum() const;  // arena bytes = max(offset + size)
  void Set(const std::string &name, size_t index, size_t size);
  const std::unordered_map<std::string, std::tuple<size_t, size_t>> &GetAll() const;

 private:
  std::unordered_map<std::string, std::tuple<size_t, size_t>> indices_;
};

class Plan {
 public:
  virtual ~Plan() = default;
  virtual Index Run(Infos &infos) const = 0;
};

// Bump allocation: each popped request goes at the current maximum (linear.cpp:5-15).
class LinearPlan : public Plan {
 public:
  Index Run(Infos &infos) const override;
};

// Best-fit over the address ranges of already placed requests whose lifetimes
// come within one step of the new one (greedy.cpp:239-270).
class GreedyPlan : public Plan {
 public:
  Index Run(Infos &infos) const override;
};

}  // namespace memory
}  // namespace fluidml

#endif
