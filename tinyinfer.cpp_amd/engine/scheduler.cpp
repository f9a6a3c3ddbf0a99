// The scheduler: which tokens of which requests the next step runs, and the loop that runs them.
//
// The reference has no scheduler: every prompt is prefilled whole in one batch and then every
// unfinished sequence decodes one token per step, in a cache sized so that nothing can run out
// (/root/reference/src/main.cpp:210-297).  Here requests wait in a queue, are admitted while a
// request slot and pages for their first portion are free, have their prompts cut into portions
// under a token budget, decode beside the portions of others, and give everything back when they
// end.
//
// Decisions, all taken in `plan()` from host bookkeeping only:
//   * every running request feeds the tokens it has not fed yet: one token if it is decoding, else
//     a portion of at most `chunk_size`; requests that decode go first (oldest first), then
//     portions of running requests, then new admissions, until `max_batched_tokens` is used up;
//   * a request's logits are wanted only at the last token it has, when the step feeds it (then
//     its next token is sampled);
//   * when the free pages cannot cover the step, the running request admitted last is preempted:
//     its pages and slot go back, it keeps its tokens (prompt and what it generated) and goes to
//     the front of the queue, to be fed again from position 0 later.  The oldest running request
//     is never preempted; if it alone cannot be covered, that is an error;
//   * a request whose prompt plus `max_new_tokens` exceeds `max_seq`, or needs more pages than the
//     pool has, is refused when it is added.
// The n-th token of a request is drawn from (seed, request number, n), so neither batching nor
// preemption changes what is sampled.
#include <algorithm>
#include <atomic>
#include <chrono>

#include "../include/inference.h"

namespace tinyinfer {

// Cache keys of the requests of different schedulers never meet: each scheduler numbers its
// requests from a base of its own.
static std::atomic<int64_t> g_next_base{int64_t(1) << 40};

Scheduler::Scheduler(CacheManager& cache_, int max_batched_tokens_, int chunk_size_, int max_running_)
    : cache(cache_), max_batched_tokens(max_batched_tokens_), chunk_size(chunk_size_) {
  if (max_batched_tokens <= 0 || chunk_size <= 0) throw SchedulerError("max_batched_tokens and chunk_size must be positive");
  max_running = std::min(cache.max_requests, max_running_ > 0 ? max_running_ : cache.max_requests);
  key_base_ = g_next_base.fetch_add(int64_t(1) << 32);
}

std::shared_ptr<Request> Scheduler::add(const std::vector<int>& prompt, int max_new_tokens, const SamplingParams& params,
                                        const std::vector<int>& eos_token_ids) {
  if (prompt.empty()) throw SchedulerError("a request needs at least one prompt token");
  if (max_new_tokens < 1) throw SchedulerError("max_new_tokens must be at least 1");
  const int total = (int)prompt.size() + max_new_tokens;
  if (total > cache.max_seq)
    throw SchedulerError("prompt (" + std::to_string(prompt.size()) + ") + max_new_tokens (" + std::to_string(max_new_tokens) +
                         ") exceeds max_seq = " + std::to_string(cache.max_seq));
  const int pages = (total + cache.page_size - 1) / cache.page_size;
  for (int g : cache.paged_groups())
    if (pages > cache.pool(g).num_pages())
      throw SchedulerError("the request needs " + std::to_string(pages) + " pages but the pool has " +
                           std::to_string(cache.pool(g).num_pages()));
  auto req = std::make_shared<Request>();
  req->number = submitted_++;
  req->key_base = key_base_;
  req->prompt = prompt;
  req->max_new_tokens = max_new_tokens;
  req->params = params;
  req->eos_token_ids = eos_token_ids;
  req->tokens = prompt;
  waiting.push_back(req);
  return req;
}

// Pages the tightest group lacks for `batch` = [(request, n_tokens)] (<= 0: it fits).
int Scheduler::new_pages(const std::vector<std::pair<std::shared_ptr<Request>, int>>& batch) const {
  if (cache.paged_groups().empty()) return 0;
  int worst = -(1 << 30);
  for (int g : cache.paged_groups()) {
    int need = 0;
    for (const auto& kv : batch) {
      const bool admitted = cache.has(kv.first->key());
      need += cache.pages_to_cover(g, kv.first->key(), admitted, kv.first->n_fed + kv.second);
    }
    worst = std::max(worst, need - const_cast<CacheManager&>(cache).pool(g).num_free());
  }
  return worst;
}

void Scheduler::preempt(const std::shared_ptr<Request>& req, Plan& plan) {
  running.erase(std::remove(running.begin(), running.end(), req), running.end());
  if (cache.has(req->key())) cache.release(req->key());
  req->n_fed = 0;
  req->preemptions += 1;
  waiting.insert(waiting.begin(), req);
  plan.preempted.push_back(req);
}

Plan Scheduler::plan() {
  Plan plan;
  std::vector<std::pair<std::shared_ptr<Request>, int>> batch;
  int budget = max_batched_tokens;
  // running requests: those that decode go first, oldest first within each kind.  If the free
  // pages cannot cover them, the one admitted last gives way and the step is planned again.
  while (true) {
    budget = max_batched_tokens;
    batch.clear();
    std::vector<std::shared_ptr<Request>> order = running;
    std::stable_sort(order.begin(), order.end(), [](const std::shared_ptr<Request>& a, const std::shared_ptr<Request>& b) {
      const bool ad = a->pending() != 1, bd = b->pending() != 1;
      if (ad != bd) return !ad;
      return a->admitted_at < b->admitted_at;
    });
    for (const auto& req : order) {
      if (budget <= 0) break;
      const int n = std::min({req->pending(), chunk_size, budget});
      batch.emplace_back(req, n);
      budget -= n;
    }
    if (batch.empty() || new_pages(batch) <= 0) break;
    if (running.size() == 1)
      throw SchedulerError("request " + std::to_string(running[0]->number) + " cannot get pages for " +
                           std::to_string(batch[0].second) + " more tokens although it is the only one running: the cache "
                           "pool is too small for it");
    auto youngest = *std::max_element(running.begin(), running.end(), [](const std::shared_ptr<Request>& a, const std::shared_ptr<Request>& b) {
      return a->admitted_at < b->admitted_at;
    });
    preempt(youngest, plan);
  }
  // admissions: in queue order, while a slot and pages for the first portion are free
  while (!waiting.empty() && budget > 0 && (int)running.size() < max_running) {
    auto req = waiting.front();
    if (std::find(plan.preempted.begin(), plan.preempted.end(), req) != plan.preempted.end()) break;   // it has just given way
    int new_in_batch = 0;
    for (const auto& kv : batch) new_in_batch += cache.has(kv.first->key()) ? 0 : 1;
    if (cache.num_free_slots() - new_in_batch <= 0) break;
    const int n = std::min({req->pending(), chunk_size, budget});
    auto with = batch;
    with.emplace_back(req, n);
    if (new_pages(with) > 0) break;
    waiting.erase(waiting.begin());
    req->admitted_at = admissions_++;
    running.push_back(req);
    batch.emplace_back(req, n);
    budget -= n;
  }
  for (const auto& kv : batch) {
    PlannedEntry e;
    e.request = kv.first;
    e.start = kv.first->n_fed;
    e.n_tokens = kv.second;
    e.sample = kv.first->n_fed + kv.second == (int)kv.first->tokens.size();
    plan.entries.push_back(e);
  }
  if (plan.entries.empty() && has_work())
    throw SchedulerError("nothing can run: the cache pool cannot take the next request's first portion");
  return plan;
}

// The step after `last`, planned before `last`'s tokens are known: possible when `last` decodes
// one token of every running request, nobody waits, none of them ends with `last`'s token by its
// length, and the pages for one more token each are free.  Every request then decodes one more
// token, whatever `last` samples; the ids come from the device (token_from_feedback).  A request
// that `last`'s token ends (an end-of-generation id) has run one token for nothing.  An empty plan
// if any of this does not hold.  Call it after `last` has been launched and before it is committed.
Plan Scheduler::plan_ahead(const Plan& last) const {
  Plan ahead;
  if (last.entries.empty() || !waiting.empty() || last.entries.size() != running.size()) return ahead;
  std::vector<std::pair<std::shared_ptr<Request>, int>> batch;
  for (const auto& e : last.entries) {
    const Request& r = *e.request;
    if (e.n_tokens != 1 || !e.sample || !r.finish_reason.empty()) return ahead;
    if (std::find(running.begin(), running.end(), e.request) == running.end()) return ahead;
    if ((int)r.generated.size() + 1 >= r.max_new_tokens) return ahead;
    batch.emplace_back(e.request, 2);           // n_fed does not count `last`'s token yet
  }
  if (new_pages(batch) > 0) return ahead;
  for (const auto& e : last.entries) {
    PlannedEntry a;
    a.request = e.request;
    a.start = e.start + 1;
    a.n_tokens = 1;
    a.sample = true;
    ahead.entries.push_back(a);
  }
  return ahead;
}

std::vector<std::shared_ptr<Request>> Scheduler::commit(const Plan& plan, const std::map<int64_t, int>& sampled) {
  std::vector<std::shared_ptr<Request>> done;
  for (const auto& e : plan.entries) {
    Request& req = *e.request;
    req.n_fed += e.n_tokens;
    if (!e.sample) continue;
    auto it = sampled.find(req.number);
    if (it == sampled.end()) throw SchedulerError("request " + std::to_string(req.number) + " asked for a token and got none");
    const int tok = it->second;
    // the reference drops an end-of-generation token instead of emitting it
    // (/root/reference/src/main.cpp:255,287) and counts the first token from the prefill step
    // towards -n (main.cpp:258,284)
    if (std::find(req.eos_token_ids.begin(), req.eos_token_ids.end(), tok) != req.eos_token_ids.end()) {
      req.finish_reason = "eos";
    } else {
      req.generated.push_back(tok);
      req.tokens.push_back(tok);
      if ((int)req.generated.size() >= req.max_new_tokens) req.finish_reason = "length";
    }
    if (!req.finish_reason.empty()) done.push_back(e.request);
  }
  for (const auto& r : done) {
    running.erase(std::remove(running.begin(), running.end(), r), running.end());
    finished.push_back(r);
  }
  return done;
}

void Scheduler::abort(const std::shared_ptr<Request>& req) {
  running.erase(std::remove(running.begin(), running.end(), req), running.end());
  waiting.erase(std::remove(waiting.begin(), waiting.end(), req), waiting.end());
  if (cache.has(req->key())) cache.release(req->key());
  if (req->finish_reason.empty()) {
    req->finish_reason = "abort";
    finished.push_back(req);
  }
}

void Scheduler::abort_all() {
  auto all = running;
  all.insert(all.end(), waiting.begin(), waiting.end());
  for (const auto& r : all) abort(r);
}

// The loop of /root/reference/src/main.cpp:210-297 with admission, portions and preemption added.
void run_requests(Engine& engine, Scheduler& scheduler, Sampler* sampler, GenerationStats* stats,
                  const std::function<void(const Request&, int)>& on_token, bool use_graph, bool run_ahead,
                  const PromptLogits& on_prompt_logits) {
  std::unique_ptr<Sampler> own;
  if (!sampler) {
    own.reset(new Sampler(engine.ops));
    sampler = own.get();
  }
  GenerationStats local;
  GenerationStats& st = stats ? *stats : local;
  // A step that has been launched and not yet read.
  struct Launched {
    Plan plan;
    std::vector<std::shared_ptr<Request>> asked;     // row i of the sampler's call
    uint64_t ticket = 0;
    bool sampled = false, decode_only = true;
    int64_t n_tok = 0;
  };
  int* feedback = run_ahead ? engine.token_feedback() : nullptr;
  std::unique_ptr<Launched> flying, next;

  // `before`: the step whose ids this one takes from the device (null: it has every id on the host)
  auto launch = [&](Plan plan, const Launched* before) {
    std::unique_ptr<Launched> f(new Launched());
    std::map<int64_t, int> row_before;
    if (before)
      for (size_t i = 0; i < before->asked.size(); ++i) row_before[before->asked[i]->number] = (int)i;
    std::vector<StepEntry> entries;
    entries.reserve(plan.entries.size());
    for (const auto& e : plan.entries) {
      StepEntry se;
      se.request = e.request->key();
      if (before)
        se.tokens.assign(1, token_from_feedback(row_before.at(e.request->number)));
      else
        se.tokens.assign(e.request->tokens.begin() + e.start, e.request->tokens.begin() + e.start + e.n_tokens);
      if (e.sample) se.want.push_back(e.n_tokens - 1);
      se.start = e.start;
      entries.push_back(std::move(se));
      f->decode_only = f->decode_only && e.n_tokens == 1;
      f->n_tok += e.n_tokens;
      if (e.sample) f->asked.push_back(e.request);
    }
    Tensor logits = use_graph ? engine.step_graph(entries) : engine.step(entries);
    if (on_prompt_logits && !before && logits.defined()) {
      // rows of requests whose prompt this step finishes
      std::vector<float> host;
      for (size_t i = 0; i < f->asked.size(); ++i) {
        if (!f->asked[i]->generated.empty()) continue;
        if (host.empty()) {
          host.resize((size_t)logits.numel());
          engine.logits_to_host(logits, host.data());
        }
        on_prompt_logits(*f->asked[i], host.data() + i * (size_t)logits.shape[1], logits.shape[1]);
      }
    }
    if (!f->asked.empty()) {
      std::vector<SamplingParams> params;
      std::vector<int64_t> numbers, counters;
      for (const auto& r : f->asked) {
        params.push_back(r->params);
        numbers.push_back(r->number);
        counters.push_back((int64_t)r->generated.size() + (before ? 1 : 0));
      }
      const bool feed = feedback && (int)f->asked.size() <= engine.feedback_rows();
      f->ticket = sampler->sample_async(logits, params, numbers, counters, feed ? feedback : nullptr);
      f->sampled = true;
    }
    f->plan = std::move(plan);
    return f;
  };

  auto t_mark = std::chrono::steady_clock::now();
  // read the step's ids, commit them, give back what ended
  auto settle = [&](Launched& f) {
    std::map<int64_t, int> sampled;
    if (f.sampled) {
      f.sampled = false;
      const std::vector<int> toks = sampler->collect(f.ticket);
      for (size_t i = 0; i < f.asked.size(); ++i) sampled[f.asked[i]->number] = toks[i];
    } else {
      engine.synchronize();
    }
    const auto now = std::chrono::steady_clock::now();
    const double ms = std::chrono::duration<double, std::milli>(now - t_mark).count();
    t_mark = now;
    if (f.decode_only) {
      st.decode_ms += ms;
      st.decode_tokens += f.n_tok;
    } else {
      st.prefill_ms += ms;
      st.prefill_tokens += f.n_tok;
    }
    st.steps += 1;
    // a step launched ahead may hold requests that the step before it ended: their row ran for nothing
    Plan live;
    live.preempted = f.plan.preempted;
    for (const auto& e : f.plan.entries)
      if (e.request->finish_reason.empty()) live.entries.push_back(e);
    std::map<int64_t, size_t> had;
    for (const auto& e : live.entries) had[e.request->number] = e.request->generated.size();
    for (const auto& done : scheduler.commit(live, sampled)) engine.release(done->key());
    if (on_token)
      for (const auto& e : live.entries)
        if (e.sample && e.request->generated.size() > had[e.request->number]) on_token(*e.request, e.request->generated.back());
  };

  try {
    while (flying || scheduler.has_work()) {
      if (!flying) {
        Plan plan = scheduler.plan();
        st.preemptions += (int64_t)plan.preempted.size();
        flying = launch(std::move(plan), nullptr);
      }
      // while the device works on that step: the next one, if it needs nothing the step decides
      if (feedback && flying->sampled && (int)flying->asked.size() <= engine.feedback_rows()) {
        Plan ahead = scheduler.plan_ahead(flying->plan);
        if (!ahead.entries.empty()) {
          try {
            next = launch(std::move(ahead), flying.get());
            st.steps_ahead += 1;
          } catch (const OutOfPages&) {
            next.reset();                    // the step has taken nothing: decided again once this one is read
          }
        }
      }
      settle(*flying);
      flying = std::move(next);
      next.reset();
    }
  } catch (...) {
    for (auto* f : {flying.get(), next.get()})
      if (f && f->sampled) sampler->drop(f->ticket);
    // whatever the scheduler still holds goes back to the cache: the next call starts clean
    scheduler.abort_all();
    throw;
  }
}

std::vector<std::vector<int>> generate(Engine& engine, const std::vector<std::vector<int>>& prompts,
                                       const GenerateOptions& o, GenerationStats* stats) {
  std::vector<int> eos = o.eos_token_ids;
  if (eos.empty() && o.use_model_eos)
    for (int64_t e : engine.model->spec.eos_token_ids) eos.push_back((int)e);
  Scheduler scheduler(*engine.cache, o.max_batched_tokens, o.chunk_size);
  std::vector<std::shared_ptr<Request>> requests;
  for (const auto& p : prompts) requests.push_back(scheduler.add(p, o.max_new_tokens, o.sampling, eos));
  run_requests(engine, scheduler, nullptr, stats, nullptr, o.use_graph, o.run_ahead);
  std::vector<std::vector<int>> out;
  for (const auto& r : requests) out.push_back(r->generated);
  return out;
}

}  // namespace tinyinfer
