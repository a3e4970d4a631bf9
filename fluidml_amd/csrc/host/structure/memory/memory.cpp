#include "structure/memory/memory.h"

#include <algorithm>
#include <stdexcept>

namespace fluidml {
namespace memory {

Info::Info(std::string &&name, size_t start, size_t end, size_t size)
    : name_(std::move(name)), start_(start), end_(end), size_(size) {}
const std::string &Info::GetName() const { return name_; }
size_t Info::GetStart() const { return start_; }
size_t Info::GetEnd() const { return end_; }
size_t Info::GetSize() const { return size_; }

bool PlainInfos::IsEmpty() const { return infos_.empty(); }
void PlainInfos::Push(Info &&info) { infos_.push_back(std::move(info)); }
Info PlainInfos::Pop() {
  if (infos_.empty()) throw std::out_of_range("PlainInfos::Pop on an empty queue");
  Info info = std::move(infos_.front());
  infos_.pop_front();
  return info;
}

bool GreedyInfos::InfoCompare::operator()(const Info &lhs, const Info &rhs) const {
  return lhs.GetSize() < rhs.GetSize();
}
bool GreedyInfos::IsEmpty() const { return infos_.empty(); }
void GreedyInfos::Push(Info &&info) { infos_.push(std::move(info)); }
Info GreedyInfos::Pop() {
  if (infos_.empty()) throw std::out_of_range("GreedyInfos::Pop on an empty queue");
  Info info = infos_.top();
  infos_.pop();
  return info;
}

size_t Index::Get(const std::string &name) const { return std::get<0>(indices_.at(name)); }
bool Index::Has(const std::string &name) const { return indices_.find(name) != indices_.end(); }
size_t Index::GetSize(const std::string &name) const { return std::get<1>(indices_.at(name)); }
size_t Index::GetMaximum() const {
  size_t maximum = 0;
  for (const auto &entry : indices_) {
    maximum = std::max(maximum, std::get<0>(entry.second) + std::get<1>(entry.second));
  }
  return maximum;
}
void Index::Set(const std::string &name, size_t index, size_t size) {
  indices_.insert({name, std::make_tuple(index, size)});
}
const std::unordered_map<std::string, std::tuple<size_t, size_t>> &Index::GetAll() const { return indices_; }

Index LinearPlan::Run(Infos &infos) const {
  Index index;
  while (!infos.IsEmpty()) {
    Info info = infos.Pop();
    index.Set(info.GetName(), index.GetMaximum(), info.GetSize());
  }
  return index;
}

namespace {

// A placed request: its bytes [lo, hi) and its widened lifetime.
struct Placed {
  size_t lo, hi;
  size_t life_lo, life_hi;
};

// The address ranges that are taken while the new request is alive, kept as an
// ascending list of [lo, hi) runs.  The reference keeps the same list as a
// linked chain (greedy.cpp:34-55); the update rules below are its, branch for
// branch, because the chain it builds is not always the plain union of the
// inputs and the gaps of that chain are what the allocator sees.
class TakenRuns {
 public:
  void Take(size_t lo, size_t hi);
  size_t Fit(size_t size) const;

 private:
  struct Run {
    size_t lo, hi;
  };
  std::vector<Run> runs_;
};

void TakenRuns::Take(size_t lo, size_t hi) {
  if (lo >= hi) return;  // empty range: nothing taken (greedy.cpp:98-100)
  if (runs_.empty()) {
    runs_.push_back({lo, hi});
    return;
  }
  Run &first = runs_.front();
  if (hi < first.lo) {
    // strictly below the first run: new first run (greedy.cpp:102-107)
    runs_.insert(runs_.begin(), {lo, hi});
    return;
  }
  if (lo <= first.hi && hi >= first.lo) {
    // touches or overlaps the first run: widen it, then swallow AT MOST ONE
    // successor, and take that successor's end as is (greedy.cpp:108-116)
    first.lo = std::min(first.lo, lo);
    first.hi = std::max(first.hi, hi);
    if (runs_.size() > 1 && runs_[1].lo <= hi) {
      first.hi = runs_[1].hi;
      runs_.erase(runs_.begin() + 1);
    }
    return;
  }
  // here lo > first.hi (greedy.cpp:117-161): find the first run `cur` whose
  // successor ends at or after `lo` (or that has no successor)
  size_t cur = 0;
  while (cur + 1 < runs_.size() && runs_[cur + 1].hi < lo) ++cur;
  // swallow every following run that starts strictly below `hi`
  size_t next = cur + 1;
  while (next < runs_.size() && runs_[next].lo < hi) {
    lo = std::min(lo, runs_[next].lo);
    hi = std::max(hi, runs_[next].hi);
    ++next;
  }
  const bool has_next = next < runs_.size();
  const bool next_apart = !has_next || runs_[next].lo > hi;  // successor absent or strictly above
  if (next_apart && runs_[cur].hi >= lo) {
    runs_[cur].hi = hi;  // (greedy.cpp:135-138)
    runs_.erase(runs_.begin() + cur + 1, runs_.begin() + next);
  } else if (has_next && runs_[next].lo <= hi && runs_[cur].hi < lo) {
    runs_[next].lo = lo;  // successor starts exactly at `hi`: extend it downwards (greedy.cpp:139-141)
    runs_.erase(runs_.begin() + cur + 1, runs_.begin() + next);
  } else if (next_apart && runs_[cur].hi < lo) {
    runs_.erase(runs_.begin() + cur + 1, runs_.begin() + next);  // (greedy.cpp:142-148)
    runs_.insert(runs_.begin() + cur + 1, {lo, hi});
  } else if (has_next && runs_[cur].hi >= lo && runs_[next].lo <= hi) {
    runs_[cur].hi = runs_[next].hi;  // bridges cur and the successor (greedy.cpp:149-151)
    runs_.erase(runs_.begin() + cur + 1, runs_.begin() + next + 1);
  } else {
    throw std::logic_error("TakenRuns::Take: inconsistent run list");
  }
}

// Smallest gap BETWEEN two runs that holds `size` (first one wins on a tie);
// only when no such gap exists, the address right after the last run.  The
// space below the first run is never offered (greedy.cpp:176-207).  Gap widths
// are computed in size_t, like the reference.
size_t TakenRuns::Fit(size_t size) const {
  if (runs_.empty()) return 0;
  size_t where = static_cast<size_t>(-1), best = static_cast<size_t>(-1);
  for (size_t i = 0; i < runs_.size(); ++i) {
    if (i + 1 < runs_.size()) {
      const size_t gap = runs_[i + 1].lo - runs_[i].hi;
      if (gap >= size && gap < best) {
        where = runs_[i].hi;
        best = gap;
      }
    } else if (best == static_cast<size_t>(-1)) {
      where = runs_[i].hi;
    }
  }
  return where;
}

}  // namespace

Index GreedyPlan::Run(Infos &infos) const {
  Index index;
  std::vector<Placed> placed;
  while (!infos.IsEmpty()) {
    const Info current = infos.Pop();
    // lifetimes are compared one step wider than stated, on both sides of the
    // test (greedy.cpp:246-248 with :65)
    const size_t life_lo = current.GetStart(), life_hi = current.GetEnd() + 1;
    TakenRuns taken;
    for (const Placed &p : placed) {
      if (p.life_lo <= life_hi && p.life_hi >= life_lo) taken.Take(p.lo, p.hi);
    }
    const size_t at = taken.Fit(current.GetSize());
    placed.push_back({at, at + current.GetSize(), life_lo, life_hi});
    index.Set(current.GetName(), at, current.GetSize());
  }
  return index;
}

}  // namespace memory
}  // namespace fluidml
