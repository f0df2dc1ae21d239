// A log of work records that is pruned by completion marks.  Host-only, no HIP types: the mark is whatever the
// owner uses to ask "has everything queued before this point finished?" (in the library the generation and grid
// of a barrier launch, checked against the words its workgroups leave in host memory; an integer in the unit test).
//
// Use: add() a record for each piece of queued work that may have to be repeated, mark() after the launches of a
// call, prune() at the start of the next call.  prune() asks, oldest mark first, whether the mark has been
// reached, stops at the first that has not, THEN asks whether the stream is healthy, and only if it is drops the
// records the reached marks cover.  The order matters: a failure raised by work in front of a reached mark is
// visible to the health check that follows, so records are only dropped for work that is known to have finished
// well; after a failure nothing is dropped and the records left are exactly those newer than the last mark that was
// seen good - the ones a repair has to repeat.  Records of finished calls therefore never outlive the next call,
// and the log never names buffers a caller may have freed since.
#pragma once
#include <cstddef>
#include <deque>
#include <utility>
#include <vector>

namespace hpx {

template <typename Rec, typename Mark>
class CompletionLog {
 public:
  void add(const Rec& r) { recs_.push_back(r); }
  // `m` will be reached when everything added so far has finished.  Nothing new since the last mark: `m` is handed
  // back to `recycle` at once.
  template <typename Recycle>
  void mark(Mark m, Recycle recycle) {
    const size_t upto = base_ + recs_.size();
    if (!marks_.empty() && marks_.back().second == upto) { recycle(m); return; }
    if (marks_.empty() && recs_.empty()) { recycle(m); return; }
    marks_.emplace_back(m, upto);
  }
  // Returns the number of records dropped.
  template <typename Reached, typename Healthy, typename Recycle>
  size_t prune(Reached reached, Healthy healthy, Recycle recycle) {
    size_t n_marks = 0;
    while (n_marks < marks_.size() && reached(marks_[n_marks].first)) n_marks++;
    if (n_marks == 0 || !healthy()) return 0;
    const size_t upto = marks_[n_marks - 1].second;
    const size_t drop = upto - base_;
    recs_.erase(recs_.begin(), recs_.begin() + std::ptrdiff_t(drop));
    base_ = upto;
    for (size_t i = 0; i < n_marks; i++) recycle(marks_[i].first);
    marks_.erase(marks_.begin(), marks_.begin() + std::ptrdiff_t(n_marks));
    return drop;
  }
  // Everything is known to have finished (the owner waited for the stream), or has been taken over by a repair.
  template <typename Recycle>
  void clear(Recycle recycle) {
    base_ += recs_.size();
    recs_.clear();
    for (auto& m : marks_) recycle(m.first);
    marks_.clear();
  }
  const std::vector<Rec>& records() const { return recs_; }
  size_t size() const { return recs_.size(); }
  bool empty() const { return recs_.empty(); }
  size_t pending_marks() const { return marks_.size(); }

 private:
  std::vector<Rec> recs_;
  size_t base_ = 0;                              // records dropped so far: marks count in absolute positions
  std::deque<std::pair<Mark, size_t>> marks_;    // (mark, absolute position of the first record behind it)
};

}  // namespace hpx
