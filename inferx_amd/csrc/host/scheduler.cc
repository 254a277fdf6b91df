// The scheduler: all policy, no GPU.  It decides who runs, in which portions,
// and what gives when pages run out.  Part of libinferx_host.so; it drives the
// cache manager of cache.cc through that file's C interface.
//
// Policies are the reference's (src/scheduler/scheduler.cc):
//   admission   first come first served while fewer than `max_running` run; pages
//               for the whole prompt are reserved; on a shortage the request stays
//               at the head of the queue and admission stops (:294-370)
//   budget      at most `max_batch_tokens` tokens a step; sequences with one
//               pending token (decodes, last one-token portions) first, then
//               prompts in running order take min(pending, budget) (:255-291)
//   pages out   for a running sequence: the most recently admitted sequence is
//               preempted (pages back, starts over with prompt + generated tokens,
//               head of the queue); if the requester is the newest, the next
//               newest yields; if it runs alone it finishes out_of_memory
//               (:444-510, :206-229)
//   context     a sequence that would pass `max_seq_len` finishes context_limit
//   finishing   stop token (kept in the output), max_tokens, cancel (:677-758)
// Pages go back the moment a sequence finishes or is preempted (:231-245).
#include <algorithm>
#include <cstdint>
#include <deque>
#include <memory>
#include <string>
#include <vector>

extern "C" {
int ixh_cache_add(void* h, int64_t rid);
int ixh_cache_free(void* h, int64_t rid);
int ixh_cache_reserve(void* h, int64_t rid, int64_t new_len);
int ixh_cache_commit(void* h, int64_t rid, int64_t tokens);
int64_t ixh_cache_cached(void* h, int64_t rid);
int ixh_cache_contains(void* h, int64_t rid);
int ixh_cache_can_add(void* h);
}

namespace {

enum Reserve { kOk = 0, kPoolEmpty = 1, kContextFull = 2 };  // what ixh_cache_reserve returns
enum Finish { kStop = 0, kLength = 1, kCancelled = 2, kContext = 3, kOutOfMemory = 4 };

struct Seq {
  int64_t rid = 0;
  std::vector<int32_t> tokens;
  int32_t prompt_len = 0;
  int64_t max_tokens = 0, min_tokens = 0;
  std::vector<int32_t> stop;
  bool cancelled = false;
  bool pending = false;  // its last token stands for a value that is still being sampled (see launched / resolve)
  bool closing = false;  // it ends when that value arrives, whatever it is: plans leave it out
  int close_reason = 0;
  int64_t draws = 0;  // sampled tokens so far: the counter of this request's random stream
  int64_t generated() const { return static_cast<int64_t>(tokens.size()) - prompt_len; }
};

struct Done {
  int64_t rid;
  int reason;
  std::vector<int32_t> output;
};

struct Part {  // one sequence's share of a step
  Seq* seq;
  int64_t first;
  int32_t count;
  bool samples;
};

struct Sched {
  void* cache;
  int max_running;
  int64_t max_batch_tokens, max_seq_len;
  std::deque<std::unique_ptr<Seq>> waiting;
  std::vector<std::unique_ptr<Seq>> running;
  std::vector<Done> completed;
  std::vector<Part> plan;
  bool planned = false;
  std::vector<Seq*> inflight;  // the sampling sequences of the step that was launched and not yet resolved
  bool launched_step = false;
  int64_t preemptions = 0;
  std::string error;

  int64_t pending(const Seq& s) const { return static_cast<int64_t>(s.tokens.size()) - ixh_cache_cached(cache, s.rid); }

  void retire(std::unique_ptr<Seq> s, int reason) {
    completed.push_back({s->rid, reason, std::vector<int32_t>(s->tokens.begin() + s->prompt_len, s->tokens.end())});
    if (ixh_cache_contains(cache, s->rid)) ixh_cache_free(cache, s->rid);
  }

  // A sequence whose sampled value is still on its way cannot be let go yet: it is marked and ends at resolve.
  void retire_or_close(size_t index, int reason) {
    if (running[index]->pending) {
      running[index]->closing = true;
      running[index]->close_reason = reason;
      return;
    }
    std::unique_ptr<Seq> gone = std::move(running[index]);
    running.erase(running.begin() + static_cast<std::ptrdiff_t>(index));
    retire(std::move(gone), reason);
  }

  void preempt(size_t index) {
    std::unique_ptr<Seq> victim = std::move(running[index]);
    running.erase(running.begin() + static_cast<std::ptrdiff_t>(index));
    ixh_cache_free(cache, victim->rid);
    waiting.push_front(std::move(victim));
    ++preemptions;
  }

  void admit() {
    while (!waiting.empty() && static_cast<int>(running.size()) < max_running) {
      Seq& s = *waiting.front();
      if (s.pending) return;  // preempted while its sampled value was on its way: it waits for that
      if (s.cancelled || static_cast<int64_t>(s.tokens.size()) > max_seq_len) {
        const int reason = s.cancelled ? kCancelled : kOutOfMemory;
        std::unique_ptr<Seq> gone = std::move(waiting.front());
        waiting.pop_front();
        retire(std::move(gone), reason);
        continue;
      }
      if (!ixh_cache_can_add(cache)) return;
      ixh_cache_add(cache, s.rid);
      const int status = ixh_cache_reserve(cache, s.rid, static_cast<int64_t>(s.tokens.size()));
      if (status != kOk) {
        ixh_cache_free(cache, s.rid);
        // Not a preemption site: it waits at the head of the queue for a running sequence to end.  With nothing
        // running nobody will ever give a page back (and a context that is too long never gets shorter), so it
        // ends here instead of being planned for ever (reference: tests/unit/scheduler_test.cc:963-984).
        if (status != kContextFull && !running.empty()) return;
        std::unique_ptr<Seq> gone = std::move(waiting.front());
        waiting.pop_front();
        retire(std::move(gone), status == kContextFull ? kContext : kOutOfMemory);
        continue;
      }
      running.push_back(std::move(waiting.front()));
      waiting.pop_front();
    }
  }

  std::vector<int64_t> take() const {
    std::vector<int64_t> t(running.size(), 0), pend(running.size(), 0);
    int64_t budget = max_batch_tokens;
    for (size_t i = 0; i < running.size(); ++i) {
      pend[i] = running[i]->closing ? 0 : pending(*running[i]);
      if (budget > 0 && pend[i] == 1) {
        t[i] = 1;
        --budget;
      }
    }
    for (size_t i = 0; i < running.size(); ++i)
      if (budget > 0 && pend[i] > 1) {
        t[i] = std::min(pend[i], budget);
        budget -= t[i];
      }
    return t;
  }

  // number of contributions (0: nothing can run), -1: called twice without a commit
  int prepare() {
    if (planned) {
      error = "prepare_step called twice without commit_step";
      return -1;
    }
    for (size_t i = 0; i < running.size();) {
      if (running[i]->cancelled && !running[i]->closing) {
        const size_t before = running.size();
        retire_or_close(i, kCancelled);
        if (running.size() == before) ++i;  // it is in flight and stays until its value has arrived
      } else {
        ++i;
      }
    }
    admit();
    std::vector<int64_t> t;
    const size_t rounds = running.size() + 1;
    for (size_t round = 0; round < rounds; ++round) {
      if (running.empty()) return 0;
      t = take();
      bool replan = false;
      for (size_t i = 0; i < running.size(); ++i) {
        if (t[i] == 0) continue;
        Seq& s = *running[i];
        const int status = ixh_cache_reserve(cache, s.rid, ixh_cache_cached(cache, s.rid) + t[i]);
        if (status == kOk) continue;
        if (status == kContextFull) {
          retire_or_close(i, kContext);
        } else {
          size_t victim = running.size() - 1;
          if (victim == i) {
            if (running.size() == 1) {
              retire_or_close(i, kOutOfMemory);
              replan = true;
              break;
            }
            victim = running.size() - 2;
          }
          preempt(victim);
        }
        replan = true;
        break;
      }
      if (!replan) break;
    }
    if (running.empty()) return 0;
    plan.clear();
    for (size_t i = 0; i < running.size(); ++i) {
      if (i >= t.size() || t[i] == 0) continue;
      Seq& s = *running[i];
      const int64_t at = ixh_cache_cached(cache, s.rid);
      plan.push_back({&s, at, static_cast<int32_t>(t[i]), at + t[i] == static_cast<int64_t>(s.tokens.size())});
    }
    if (plan.empty()) return 0;
    planned = true;
    return static_cast<int>(plan.size());
  }

  // The step has been handed to the device: what it wrote to the cache counts from now on, and every sequence that
  // samples gets a place for the value that is on its way.  Another step may be planned (prepare) before that
  // value is known; it is launched only after resolve.  Returns the number of values resolve will want.
  int launched() {
    if (!planned) {
      error = "launched without prepare_step";
      return -1;
    }
    if (launched_step) {
      error = "launched twice without resolve";
      return -2;
    }
    planned = false;
    launched_step = true;
    inflight.clear();
    for (const Part& p : plan) {
      Seq& s = *p.seq;
      ixh_cache_commit(cache, s.rid, p.count);
      if (!p.samples) continue;
      s.tokens.push_back(-1);
      ++s.draws;
      s.pending = true;
      if (!s.closing && s.generated() >= s.max_tokens) {
        s.closing = true;
        s.close_reason = kLength;
      }
      inflight.push_back(&s);
    }
    plan.clear();
    return static_cast<int>(inflight.size());
  }

  // The sampled values of the launched step, in the order of its sampling sequences.  Sequences that end (stop
  // token, length, or an ending put off while they were in flight) are let go.  Returns 1 if a step planned
  // meanwhile named one of them (that plan is dropped: prepare again), 0 otherwise.
  int resolve(const int32_t* sampled, int n) {
    if (!launched_step) {
      error = "resolve without a launched step";
      return -1;
    }
    if (n != static_cast<int>(inflight.size())) {
      error = std::to_string(n) + " sampled tokens for " + std::to_string(inflight.size()) + " sampling rows";
      return -2;
    }
    launched_step = false;
    std::vector<std::pair<Seq*, int>> finished;
    for (int i = 0; i < n; ++i) {
      Seq& s = *inflight[static_cast<size_t>(i)];
      const int32_t token = sampled[i];
      s.tokens.back() = token;
      s.pending = false;
      const bool is_stop = std::find(s.stop.begin(), s.stop.end(), token) != s.stop.end();
      if (is_stop && s.generated() > s.min_tokens)
        finished.push_back({&s, kStop});
      else if (s.generated() >= s.max_tokens)
        finished.push_back({&s, kLength});
      else if (s.closing)
        finished.push_back({&s, s.close_reason});
      s.closing = false;
    }
    inflight.clear();
    int stale = 0;
    if (planned)
      for (auto& f : finished)
        for (const Part& p : plan)
          if (p.seq == f.first) stale = 1;
    if (stale) {
      planned = false;
      plan.clear();
    }
    for (auto& f : finished) {
      bool gone_from_running = false;
      for (size_t i = 0; i < running.size(); ++i)
        if (running[i].get() == f.first) {
          std::unique_ptr<Seq> gone = std::move(running[i]);
          running.erase(running.begin() + static_cast<std::ptrdiff_t>(i));
          retire(std::move(gone), f.second);
          gone_from_running = true;
          break;
        }
      if (gone_from_running) continue;
      for (size_t i = 0; i < waiting.size(); ++i)  // it was preempted while its value was on its way
        if (waiting[i].get() == f.first) {
          std::unique_ptr<Seq> gone = std::move(waiting[i]);
          waiting.erase(waiting.begin() + static_cast<std::ptrdiff_t>(i));
          retire(std::move(gone), f.second);
          break;
        }
    }
    return stale;
  }

  // launched and resolve in one: the step has run and its values are known
  int commit(const int32_t* sampled, int n) {
    if (!planned) {
      error = "commit_step without prepare_step";
      return -1;
    }
    int want = 0;
    for (const Part& p : plan) want += p.samples ? 1 : 0;
    if (n != want) {
      error = std::to_string(n) + " sampled tokens for " + std::to_string(want) + " sampling rows";
      return -2;
    }
    const int rc = launched();
    if (rc < 0) return rc;
    return resolve(sampled, n) < 0 ? -3 : 0;
  }

  Seq* find(int64_t rid) {
    for (auto& s : running)
      if (s->rid == rid) return s.get();
    for (auto& s : waiting)
      if (s->rid == rid) return s.get();
    return nullptr;
  }
};

Sched* S(void* h) { return static_cast<Sched*>(h); }

}  // namespace

extern "C" {

void* ixh_sched_create(void* cache, int max_running, int64_t max_batch_tokens, int64_t max_seq_len) {
  if (cache == nullptr || max_running <= 0 || max_batch_tokens <= 0 || max_seq_len <= 0) return nullptr;
  Sched* s = new Sched();
  s->cache = cache;
  s->max_running = max_running;
  s->max_batch_tokens = max_batch_tokens;
  s->max_seq_len = max_seq_len;
  return s;
}
void ixh_sched_destroy(void* h) { delete S(h); }
const char* ixh_sched_error(void* h) { return S(h)->error.c_str(); }

// 0 ok, -1 empty prompt, -2 the request is already known
int ixh_sched_add(void* h, int64_t rid, const int32_t* prompt, int n, int64_t max_tokens, int64_t min_tokens,
                  const int32_t* stop, int n_stop) {
  if (n <= 0) return -1;
  if (S(h)->find(rid) != nullptr) return -2;
  std::unique_ptr<Seq> s(new Seq());
  s->rid = rid;
  s->tokens.assign(prompt, prompt + n);
  s->prompt_len = n;
  s->max_tokens = max_tokens;
  s->min_tokens = min_tokens;
  if (n_stop > 0) s->stop.assign(stop, stop + n_stop);
  S(h)->waiting.push_back(std::move(s));
  return 0;
}
void ixh_sched_cancel(void* h, int64_t rid) {
  if (Seq* s = S(h)->find(rid)) s->cancelled = true;
}
int ixh_sched_has_work(void* h) { return (!S(h)->waiting.empty() || !S(h)->running.empty()) ? 1 : 0; }
int64_t ixh_sched_preemptions(void* h) { return S(h)->preemptions; }

int ixh_sched_prepare(void* h) { return S(h)->prepare(); }
int64_t ixh_sched_plan_tokens(void* h) {
  int64_t n = 0;
  for (const Part& p : S(h)->plan) n += p.count;
  return n;
}
// the plan of the step: per contribution the request, its first position, its number of tokens, whether its last
// row gives the next token, and (flat, `tokens` with room for ixh_sched_plan_tokens numbers) the tokens
void ixh_sched_plan(void* h, int64_t* rids, int64_t* first, int32_t* counts, int32_t* samples, int32_t* tokens) {
  size_t at = 0, i = 0;
  for (const Part& p : S(h)->plan) {
    rids[i] = p.seq->rid;
    first[i] = p.first;
    counts[i] = p.count;
    samples[i] = p.samples ? 1 : 0;
    std::copy(p.seq->tokens.begin() + p.first, p.seq->tokens.begin() + p.first + p.count, tokens + at);
    at += static_cast<size_t>(p.count);
    ++i;
  }
}
int ixh_sched_commit(void* h, const int32_t* sampled, int n) { return S(h)->commit(sampled, n); }
int ixh_sched_launched(void* h) { return S(h)->launched(); }
int ixh_sched_resolve(void* h, const int32_t* sampled, int n) { return S(h)->resolve(sampled, n); }
int ixh_sched_is_planned(void* h) { return S(h)->planned ? 1 : 0; }
// The planned step will not run after all (its launch failed): the plan is dropped, the pages it reserved stay
// with their sequences, and the next prepare plans afresh.
void ixh_sched_abandon(void* h) {
  S(h)->planned = false;
  S(h)->plan.clear();
}
// the tokens of the planned step again (flat, as ixh_sched_plan gives them): after resolve they are all known
void ixh_sched_plan_token_values(void* h, int32_t* tokens) {
  size_t at = 0;
  for (const Part& p : S(h)->plan) {
    std::copy(p.seq->tokens.begin() + p.first, p.seq->tokens.begin() + p.first + p.count, tokens + at);
    at += static_cast<size_t>(p.count);
  }
}

int ixh_sched_num_completed(void* h) { return static_cast<int>(S(h)->completed.size()); }
void ixh_sched_completed(void* h, int i, int64_t* rid, int32_t* reason, int32_t* n_out) {
  const Done& d = S(h)->completed[static_cast<size_t>(i)];
  *rid = d.rid;
  *reason = d.reason;
  *n_out = static_cast<int32_t>(d.output.size());
}
void ixh_sched_completed_tokens(void* h, int i, int32_t* out) {
  const Done& d = S(h)->completed[static_cast<size_t>(i)];
  std::copy(d.output.begin(), d.output.end(), out);
}
void ixh_sched_clear_completed(void* h) { S(h)->completed.clear(); }

// which = 0: the running sequences in order of admission, 1: the waiting ones from the head of the queue
int ixh_sched_list(void* h, int which, int64_t* out, int cap) {
  int n = 0;
  if (which == 0) {
    for (auto& s : S(h)->running)
      if (n < cap) out[n++] = s->rid;
    return static_cast<int>(S(h)->running.size());
  }
  for (auto& s : S(h)->waiting)
    if (n < cap) out[n++] = s->rid;
  return static_cast<int>(S(h)->waiting.size());
}
// 0 ok, -1 unknown request
int ixh_sched_seq_info(void* h, int64_t rid, int32_t* prompt_len, int64_t* n_tokens, int64_t* draws) {
  Seq* s = S(h)->find(rid);
  if (s == nullptr) return -1;
  *prompt_len = s->prompt_len;
  *n_tokens = static_cast<int64_t>(s->tokens.size());
  *draws = s->draws;
  return 0;
}
int ixh_sched_seq_tokens(void* h, int64_t rid, int64_t from, int32_t* out, int64_t cap) {
  Seq* s = S(h)->find(rid);
  if (s == nullptr) return -1;
  int64_t n = 0;
  for (int64_t i = from; i < static_cast<int64_t>(s->tokens.size()) && n < cap; ++i) out[n++] = s->tokens[static_cast<size_t>(i)];
  return static_cast<int>(n);
}

}  // extern "C"
