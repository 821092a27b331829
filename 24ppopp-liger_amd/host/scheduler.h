// scheduler.h -- profile-driven two-stream scheduler with hybrid (host + device event) synchronisation.
//
// Counterpart of the reference's src/schedule.h (Scheduler<T, MODEL>: profile :79-157, serve :159-172, update_vec
// :175-202, run_sequential :204-219, run_stream_sync :221-278, run_stop :280-282, request simulator :285-321,
// output_recording :325-350).  Same structure: a request thread builds launch vectors and queues Samples; the
// scheduler thread runs rounds -- the primary request launches one run of same-class kernels on stream 0, then up to
// contention_factor x (profiled time of that run) worth of other-class kernels of the waiting requests is launched
// on stream 1, splitting a GEMM when only a fraction fits.  The host blocks on an event recorded before the LAST
// kernel of the previous round (so it prepares the next round while that kernel runs) and stream 1 is gated on the
// END of the previous round by a device-side event wait.
// Differences: a mutex-protected queue and an atomic stop flag (the reference shares a std::queue and a bool between
// threads unguarded); per-request input/output/workspace/KV-cache contexts (the reference shares one set between all
// in-flight requests); the class notion is a policy (see sample.h); requests may carry decode steps; the report
// adds p99; the loop ends when stop has been requested AND all work has drained.
#pragma once
#include <cmath>
#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <deque>
#include <mutex>
#include <thread>

#include "layers.h"
#include "sample.h"

namespace liger {

// Times one launch-vector entry the way the reference's profiler does (schedule.h:93-112): two warm-up launches,
// device sync, `iters` launches between two events on the launch stream; minimum over `trials`.  Returns ms/launch.
inline float profile_callback(FuncWrap& f, const DynamicInitParam& D, void* e0, void* e1, int iters = 20, int trials = 3) {
    float best = 1e30f;
    for (int t = 0; t < trials; ++t) {
        f.callback(D);
        f.callback(D);
        note_status(lg_device_synchronize(), "lg_device_synchronize");
        note_status(lg_event_record(e0, D.stream), "lg_event_record");
        for (int i = 0; i < iters; ++i) f.callback(D);
        note_status(lg_event_record(e1, D.stream), "lg_event_record");
        note_status(lg_event_synchronize(e1), "lg_event_synchronize");
        float ms = 0.f;
        note_status(lg_event_elapsed_ms(&ms, e0, e1), "lg_event_elapsed_ms");
        if (ms < best) best = ms;
    }
    return best / (float)iters;
}

struct TraceRequest {
    double arrival_s;  // offset from the start of the trace
    int batch, seq, n_decode;
};

struct Report {
    int records = 0;
    double avg_latency_ms = 0, p99_latency_ms = 0, avg_gpu_ms = 0, avg_queue_ms = 0, total_duration_ms = 0, throughput = 0;
    // arrival -> completion on one clock (not in the reference's report): the stop event's distance from an epoch event whose
    // host time is known, minus the arrival's.  cpu + gpu time under-counts when a request's start event, launched on the
    // second stream, is held up on the device behind the first stream's work.
    double avg_e2e_ms = 0, p99_e2e_ms = 0;
};

// Pure arithmetic of the reference's report (schedule.h:325-348): latency_i = cpu_ms[i] + gpu_ms[i];
// Average Latency = mean; Throughput = 1000 * count / total_duration_ms.  p99 = nearest-rank percentile.
inline Report summarize_records(const std::vector<double>& cpu_ms, const std::vector<double>& gpu_ms, double total_duration_ms) {
    Report r;
    r.records = (int)std::min(cpu_ms.size(), gpu_ms.size());
    if (r.records == 0) return r;
    std::vector<double> lat(r.records);
    double sl = 0, sg = 0, sq = 0;
    for (int i = 0; i < r.records; ++i) {
        lat[i] = cpu_ms[i] + gpu_ms[i];
        sl += lat[i]; sg += gpu_ms[i]; sq += cpu_ms[i];
    }
    r.avg_latency_ms = sl / r.records;
    r.avg_gpu_ms = sg / r.records;
    r.avg_queue_ms = sq / r.records;
    std::sort(lat.begin(), lat.end());
    int rank = (int)std::ceil(0.99 * r.records);
    r.p99_latency_ms = lat[std::max(1, rank) - 1];
    r.total_duration_ms = total_duration_ms;
    r.throughput = total_duration_ms > 0 ? 1000.0 * r.records / total_duration_ms : 0;
    return r;
}

// Deterministic Poisson trace: exponential inter-arrival times with rate lambda (req/s), prompt lengths uniform in
// [seq_lo, seq_hi] rounded down to a multiple of seq_round (the reference rejects batch*seq % 4 != 0, schedule.h:299).
inline std::vector<TraceRequest> make_poisson_trace(double lambda, int n, int batch, int seq_lo, int seq_hi, int seq_round,
                                                    int n_decode, uint64_t seed) {
    auto next = [&seed]() {
        seed += 0x9E3779B97F4A7C15ull;
        uint64_t z = seed;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    };
    std::vector<TraceRequest> tr;
    double t = 0;
    for (int i = 0; i < n; ++i) {
        const double u = ((double)(next() >> 11) + 0.5) / 9007199254740992.0;  // (0,1)
        t += -std::log(u) / lambda;
        int s = seq_lo + (int)(next() % (uint64_t)(seq_hi - seq_lo + 1));
        if (seq_round > 1) s = std::max(seq_round, s / seq_round * seq_round);
        tr.push_back({t, batch, s, n_decode});
    }
    return tr;
}

template <class T, class MODELTYPE>
class Scheduler {
  public:
    struct ReqCtx {
        T *input, *output, *ws, *dec_a, *dec_b;
        int slot;
    };

  private:
    MODELTYPE* _model;
    std::thread _thread;
    std::mutex _q_mutex;
    std::deque<Sample*> _main_q;
    std::mutex _pool_mutex;
    std::condition_variable _pool_cv;
    std::vector<ReqCtx*> _pool;
    std::atomic<bool> _stop{false};
    int _next_id = 0;

  public:
    std::vector<Sample*> exe_vec;
    int schedule_deep = 6;            // schedule.h:30
    float contention_factor = 0.8f;   // schedule.h:249
    // Measured replacement of that constant (RESOURCE policy): contention_table[main][sub] = fraction of the stand-alone
    // time of class-`sub` kernels that is hidden when they run on stream 1 next to class-`main` kernels on stream 0.
    // Entries < 0 are unmeasured and fall back to contention_factor.
    float contention_table[3][3] = {{-1.f, -1.f, -1.f}, {-1.f, -1.f, -1.f}, {-1.f, -1.f, -1.f}};
    class_policy policy = RESOURCE;
    // RESOURCE policy: minor entries (FuncWrap::minor: normalisation, residual, cache append, row gather) take the class of
    // the entry before them, so that they neither cut a prefill into many runs nor stop an interleaved one
    bool merge_minor = false;
    split_axis axis = SPLIT_OUT_COLS;
    int seq_bucket = 1;               // durations are looked up at seq rounded up to a multiple of this
    int ignore_num = 20;              // warm-up records dropped from the report (schedule.h:327)
    int profile_misses = 0, sub_profile_misses = 0;
    int rounds = 0, secondary_launches = 0, splits = 0, partition_rounds = 0;
    // ---- spatial partition of the two streams (enable_partition) ---------------------------------------------------------
    // The reference keeps its two streams apart with stream priorities and a cap on hardware queues (schedule.h:54-55,
    // context.h:27); here a co-running round gives each class its own compute units instead: the HBM-bound side runs on
    // partition_hbm_cus of them, the MFMA-bound side on the rest, on CU-masked streams, and every kernel sizes its grid for
    // its share.  A round is partitioned only while a waiting request has work of the other class, and only for as long as
    // that work lasts; all other rounds run on the whole chip.  partition_table[main][sub] = stand-alone milliseconds of
    // class-`sub` work that complete per stand-alone millisecond of the class-`main` primary in a partitioned round
    // (measured by profile_partition; <= 0: partitioning that pair does not pay and is not done).
    // ---- decode steps of different requests as one launch vector (enable_batch_decode) ------------------------------------
    // A request's decode steps stream the whole weight shard for one token row; requests that are in their decode steps at the
    // same time therefore share one launch vector per step (per-sequence cache slots and lengths in the kernels that touch the
    // cache), which reads the weights once for all of them.  The batched step is scheduled like one more request that is always
    // last in line: the prefill of a newly arrived request goes ahead of it as the primary, the batch's HBM-bound kernels are
    // interleaved into that prefill's MFMA-bound windows, and the request joins the batch at the first step boundary after its
    // prefill.  No reference counterpart (the reference has no
    // decode phase); without it every request runs its own decode steps, as in run_sequential.
    bool batch_decode = false;
    // With batched decode steps: a single-sequence prompt longer than prefill_chunk tokens is prefilled in chunks of that many
    // (each chunk through all layers, over the request's KV-cache slot), and after every chunk the batched decode step gets the
    // primary's turn once, so that requests in their decode steps wait for a chunk, not for a whole prompt.  0 = off.
    int prefill_chunk = 0;
    int chunked_prefills = 0, yield_turns = 0;   // requests whose prefill was cut into chunks; turns given to the decode batch
    int decode_steps_ahead = 4;       // steps per batched launch vector while nothing waits to join (1 otherwise)
    int batched_steps = 0, batched_rows = 0;   // steps launched, and token rows they carried (holes included)
    // Called by the scheduler thread right after the kernels of every batched decode step have been launched, as an entry of
    // the step's launch vector (so before the rows of requests that finish with this step are copied out): the place where a
    // serving loop turns the step's hidden states into the next step's input rows (sampling + embedding), with work it puts
    // on the stream it is handed.  `step` counts the batched steps of the run; row r of the batch belongs to cache slot
    // slots[r] at pasts[r] cached positions BEFORE the step (rows of no request point at the spare slot, index
    // pool contexts x context batch).  Tests use it to check every step against the CPU oracle and to force the oracle's
    // rows into the next step.
    std::function<void(int step, const std::vector<int>& slots, const std::vector<int>& pasts, T* rows, const DynamicInitParam&)> decode_step_hook;
    T* decode_batch_rows() const { return _dec_x; }
    int partition_hbm_cus = 0;
    float partition_table[3][3] = {{-1.f, -1.f, -1.f}, {-1.f, -1.f, -1.f}, {-1.f, -1.f, -1.f}};
    float partition_min_ms = 0.05f;   // less waiting work than this is not worth a partitioned round
    // ---- does partitioning pay in THIS run?  (partition_feedback) -----------------------------------------------------------
    // partition_table comes from one measured pair of shapes in steady state; a trace has other shapes, short rounds and a host
    // synchronisation per round.  While a run is going on the scheduler therefore measures what its rounds deliver: every round
    // starts with an event on the primary's stream (behind the end of the round before it), and a round's progress rate is the
    // stand-alone milliseconds of work launched in it (primary and secondaries) per millisecond until the next round starts.
    // Rounds in which a partition is possible are run partitioned and on the whole chip in turn until both kinds have
    // partition_feedback_min samples; from then on they are partitioned only while the partitioned rounds' rate is at least
    // partition_feedback_margin times the whole-chip rounds', and every partition_feedback_probe-th such round takes the other
    // side so that both figures stay current.  The figures carry over from run to run (older samples at half weight) until the
    // share changes.  The margin is well above 1 because the estimate flatters partitioned rounds (see _round_begin): measured
    // ratios of 1.02-1.05 went with mean latencies 0.2-1.5 % behind the unpartitioned run's, ratios of 1.37-1.39 with gains.
    // No reference counterpart.
    bool partition_feedback = true;
    int partition_feedback_min = 6, partition_feedback_probe = 32;
    float partition_feedback_margin = 1.08f;
    int partition_declined = 0;       // rounds that could have been partitioned and were run on the whole chip instead
    void reset_partition_feedback() {
        for (int k = 0; k < 3; ++k) { _fb_work[k] = _fb_time[k] = 0; _fb_n[k] = 0; }
        _fb_eligible = 0;
    }
    double feedback_rate(int kind) const { return _fb_time[kind] > 0 ? _fb_work[kind] / _fb_time[kind] : 0.0; }  // 1: whole chip, 2: partitioned
    int feedback_samples(int kind) const { return _fb_n[kind]; }
    StaticInitParam SParams;
    DynamicInitParam DParams0;
    DynamicInitParam DParams1;
    MainDict profiling_res_dict;
    SubDict profiling_decompse_res_dict;
    BertInitParam BertParams;
    std::vector<recorder> recs;
    T *input, *output;  // default buffers (profile / single request), like the reference's members
    void *Main_EVENT = nullptr, *Wait_EVENT = nullptr;

    Scheduler(MODELTYPE* model, const BertInitParam& BertParams_, const StaticInitParam& SParams_, T* input_, T* output_,
              const std::string& main_filename = "", const std::string& sub_filename = "")
        : _model(model), SParams(SParams_), DParams0(-4), DParams1(0, DParams0), BertParams(BertParams_), input(input_), output(output_) {
        DParams0.stream_id = 0;
        DParams1.stream_id = 1;
        if (!main_filename.empty()) MainFileToDict(main_filename, profiling_res_dict);
        if (!sub_filename.empty()) SubFileToDict(sub_filename, profiling_decompse_res_dict);
        note_status(lg_event_create(&Main_EVENT), "lg_event_create");
        note_status(lg_event_create(&Wait_EVENT), "lg_event_create");
    }
    // Releases what the scheduler created: its streams (the two of the constructor and the CU-masked ones; every stream holds a
    // hardware queue, and queues that pile up make streams share one and run in turn), its events, the request contexts and
    // the decode batch's buffers.  The model and the buffers handed to the constructor belong to the caller.
    ~Scheduler() {
        if (_thread.joinable()) _thread.join();
        lg_device_synchronize();
        _drop_queued();
        {   // samples still in flight or retired but not yet reclaimed (none after a completed run)
            std::vector<Sample*> left(exe_vec.begin(), exe_vec.end());
            left.insert(left.end(), _retired.begin(), _retired.end());
            std::sort(left.begin(), left.end());
            left.erase(std::unique(left.begin(), left.end()), left.end());
            for (Sample* smp : left) delete smp;
        }
        _drop_partition_streams();
        DParams1.destroy();
        DParams0.destroy();
        for (void* e : {Main_EVENT, Wait_EVENT, _epoch_event, _dec_prev_stop})
            if (e) lg_event_destroy(e);
        for (RoundRec& r : _round_log) lg_event_destroy(r.begin);
        for (void* e : _round_events) lg_event_destroy(e);
        for (ReqCtx* c : _all_ctx) {
            dev_free(c->input); dev_free(c->output); dev_free(c->ws); dev_free(c->dec_a); dev_free(c->dec_b);
            delete c;
        }
        dev_free(_dec_x); dev_free(_dec_ws);
    }
    Scheduler(const Scheduler&) = delete;
    Scheduler& operator=(const Scheduler&) = delete;

    // Creates the four CU-masked streams of partitioned rounds: [role: primary, secondary] x [class: MFMA-bound, HBM-bound].
    // hbm_cus compute units (a multiple of 8, spread evenly over the 8 dies: mask bits 0 .. hbm_cus-1) go to the HBM-bound
    // side, the rest to the MFMA-bound side.  Returns false (and leaves partitioning off) on bad arguments.
    bool enable_partition(int hbm_cus, int total_cus = 256) {
        if (hbm_cus <= 0 || hbm_cus % 8 != 0 || hbm_cus >= total_cus || total_cus > 256 || total_cus % 8 != 0) return false;
        if (partition_hbm_cus == hbm_cus) return true;
        // The streams of a share are created once and kept while that share is in use (switching the partition on and off does
        // not touch them); asking for another share releases them first: every CU-masked stream is a hardware queue of its own.
        auto it = _part_streams.find(hbm_cus);
        if (it == _part_streams.end()) {
            // The error state is process-wide and sticky: with one already recorded the outcome of the stream creation below
            // could not be told apart from it, so nothing is touched and the partition in use (if any) stays as it is.
            if (first_error()) return false;
            _drop_partition_streams();
            unsigned hbm_mask[8] = {0}, mfma_mask[8] = {0};
            for (int b = 0; b < total_cus; ++b) (b < hbm_cus ? hbm_mask : mfma_mask)[b >> 5] |= 1u << (b & 31);
            PartStreams ps;
            for (int role = 0; role < 2; ++role) {
                ps.d[role][MFMA_BOUND].reset(new DynamicInitParam(mfma_mask, 8, 2 + 2 * role + MFMA_BOUND));
                ps.d[role][HBM_BOUND].reset(new DynamicInitParam(hbm_mask, 8, 2 + 2 * role + HBM_BOUND));
            }
            if (first_error()) {
                // a stream could not be created: release the ones that were (each holds a hardware queue and a workspace)
                for (int role = 0; role < 2; ++role)
                    for (int cls = 0; cls < 2; ++cls)
                        if (ps.d[role][cls]) ps.d[role][cls]->destroy();
                return false;
            }
            // The two streams of a partitioned round must sit on different hardware queues, or their kernels run strictly in
            // turn and the round is a slower sequential one.  Each (primary, secondary) pair of different classes is probed; a
            // secondary that runs in turn with its primary is replaced, the rejected candidates kept alive meanwhile so that the
            // next one is handed another queue.
            ps.verified = -1;
            if (verify_partition_streams) ps.verified = 1;
            for (int mc = 0; mc < 2 && verify_partition_streams && !first_error(); ++mc) {
                const int sc = 1 - mc;
                std::vector<std::unique_ptr<DynamicInitParam>> rejected;
                int conc = 0;
                for (int tries = 0; tries < PARTITION_STREAM_TRIES; ++tries) {
                    note_status(lg_streams_run_concurrently(ps.d[0][mc]->stream, ps.d[1][sc]->stream, &conc), "lg_streams_run_concurrently");
                    if (conc || first_error() || tries + 1 == PARTITION_STREAM_TRIES) break;
                    rejected.push_back(std::move(ps.d[1][sc]));
                    ps.d[1][sc].reset(new DynamicInitParam(sc == MFMA_BOUND ? mfma_mask : hbm_mask, 8, 2 + 2 * 1 + sc));
                    if (first_error()) break;
                }
                for (auto& r : rejected) r->destroy();
                if (!conc) ps.verified = 0;
            }
            if (first_error()) {
                for (int role = 0; role < 2; ++role)
                    for (int cls = 0; cls < 2; ++cls)
                        if (ps.d[role][cls]) ps.d[role][cls]->destroy();
                return false;
            }
            it = _part_streams.emplace(hbm_cus, std::move(ps)).first;
        }
        partition_streams_concurrent = it->second.verified;
        for (int role = 0; role < 2; ++role)
            for (int cls = 0; cls < 2; ++cls) _part[role][cls] = it->second.d[role][cls].get();
        partition_hbm_cus = hbm_cus;
        // factors measured for another share do not carry over, nor does what rounds on it delivered
        for (int a = 0; a < 3; ++a)
            for (int b = 0; b < 3; ++b) partition_table[a][b] = -1.f;
        reset_partition_feedback();
        return true;
    }
    void disable_partition() { partition_hbm_cus = 0; }
    // verify_partition_streams (set before enable_partition creates a share's streams): probe both (primary, secondary) pairs
    // for overlap and replace a secondary that takes turns with its primary.  partition_streams_concurrent: 1 both pairs were
    // measured to overlap, 0 a pair could not be made to, -1 not probed; profile_partition installs no factor at 0.  Off by
    // default: profile_partition's own measurement already rejects a share whose streams take turns (its co-run then takes
    // as long as both sides back to back: gain below 1).
    bool verify_partition_streams = false;
    int partition_streams_concurrent = -1;
    const DynamicInitParam* partition_stream(int role, int cls) const {
        return (partition_hbm_cus > 0 && (cls == MFMA_BOUND || cls == HBM_BOUND)) ? _part[role][cls] : nullptr;
    }

    // ---- per-request contexts ------------------------------------------------------------------------------
    // Allocates `count` contexts sized for (max_batch_size, max_seq_len); serve() blocks when all are in flight.
    void make_pool(int count, int ctx_batch) {
        const int H = BertParams.head_num * BertParams.size_per_head;
        const int64_t io = (int64_t)ctx_batch * BertParams.max_seq_len * H;
        const int64_t we = _model->workspace_elems(ctx_batch, BertParams.max_seq_len);
        for (int i = 0; i < count; ++i) {
            ReqCtx* c = new ReqCtx();
            c->input = dev_alloc<T>(io);
            c->output = dev_alloc<T>(io);
            c->ws = dev_alloc<T>(we);
            c->dec_a = dev_alloc<T>((int64_t)ctx_batch * H);
            c->dec_b = dev_alloc<T>((int64_t)ctx_batch * H);
            dev_fill_normal(c->dec_a, (int64_t)ctx_batch * H, 1234, 60000 + _pool_total, 0.f, 1.f);  // input of a decode-only request
            dev_fill_const(c->dec_b, (int64_t)ctx_batch * H, 0.f);
            c->slot = _pool_total * ctx_batch;
            dev_fill_normal(c->input, io, 1234, 50000 + _pool_total, 0.f, 1.f);
            _pool.push_back(c);
            _all_ctx.push_back(c);
            _pool_total++;
        }
        _ctx_batch = ctx_batch;
        note_status(lg_device_synchronize(), "lg_device_synchronize");
    }
    // Batched decode needs one more cache slot than the contexts use (rows of the batch that belong to no request in its
    // decode steps are pointed at it) and the batch's own token-row buffer and workspace.
    bool enable_batch_decode(bool on = true) {
        // batching changes what the rounds of a run look like: what partitioned rounds delivered without it says nothing about them
        if (on != batch_decode) reset_partition_feedback();
        if (!on) { batch_decode = false; return true; }
        const int rows = _pool_total * _ctx_batch;
        if (rows <= 0 || BertParams.max_cache_len <= 0 || rows + 1 > BertParams.max_batch_size || rows > LG_ATTN_DECODE_MAX_SEQS) return false;
        if (!_dec_x) {
            const int H = BertParams.head_num * BertParams.size_per_head;
            _dec_x = dev_alloc<T>((int64_t)rows * H);
            _dec_ws = dev_alloc<T>(_model->workspace_elems(rows, 1));
            note_status(lg_memset_async(_dec_x, 0, (size_t)rows * H * sizeof(T), nullptr), "lg_memset_async");
            note_status(lg_device_synchronize(), "lg_device_synchronize");
        }
        batch_decode = true;
        return first_error() == 0;
    }
    // Shapes a request may have: they decide how far the launch vector writes into the request's buffers, its workspace and
    // its KV-cache slots, so they are checked once here, on the host, before anything is built or launched.
    bool request_fits(int batch_size, int seq_len, int n_decode, const char* who) {
        const int max_b = _pool_total ? _ctx_batch : BertParams.max_batch_size;
        const bool ok = batch_size > 0 && seq_len > 0 && n_decode >= 0 && batch_size <= max_b && seq_len <= BertParams.max_seq_len &&
                        (n_decode == 0 || (BertParams.max_cache_len > 0 && seq_len + n_decode <= BertParams.max_cache_len));
        if (!ok && error_code() == 0)
            set_error_state(LG_ERR_INVALID, std::string(who) + ": request (batch " + std::to_string(batch_size) + ", seq " + std::to_string(seq_len) +
                            ", decode steps " + std::to_string(n_decode) + ") exceeds the contexts (batch " + std::to_string(max_b) + ", seq " +
                            std::to_string(BertParams.max_seq_len) + ", cache " + std::to_string(BertParams.max_cache_len) + ")");
        return ok;
    }
    bool decode_fits(int batch_size, int past, int n_steps, const char* who) {
        const int max_b = _pool_total ? _ctx_batch : BertParams.max_batch_size;
        const bool ok = batch_size > 0 && past >= 0 && n_steps > 0 && batch_size <= max_b && BertParams.max_cache_len > 0 &&
                        past + n_steps <= BertParams.max_cache_len;
        if (!ok && error_code() == 0)
            set_error_state(LG_ERR_INVALID, std::string(who) + ": decode request (batch " + std::to_string(batch_size) + ", past " + std::to_string(past) +
                            ", steps " + std::to_string(n_steps) + ") exceeds the contexts (batch " + std::to_string(max_b) + ", cache " +
                            std::to_string(BertParams.max_cache_len) + ")");
        return ok;
    }
    // contexts in creation order (tests compare a request's output buffer with a plain sequential run)
    const ReqCtx* context(int i) const { return (i >= 0 && i < (int)_all_ctx.size()) ? _all_ctx[i] : nullptr; }
    // Blocks while every context is in flight -- but only if a scheduler loop is running that can return one; with no loop
    // running (requests queued up front, more of them than contexts) it fails with nullptr instead of waiting forever.
    ReqCtx* acquire_ctx() {
        std::unique_lock<std::mutex> lk(_pool_mutex);
        _pool_cv.wait(lk, [this] { return !_pool.empty() || !_running.load(); });
        if (_pool.empty()) return nullptr;
        // the free context with the lowest cache slot: the rows of a batched decode step then stay dense
        size_t pick = 0;
        for (size_t i = 1; i < _pool.size(); ++i)
            if (_pool[i]->slot < _pool[pick]->slot) pick = i;
        ReqCtx* c = _pool[pick];
        _pool.erase(_pool.begin() + pick);
        return c;
    }
    // recycle_contexts = false keeps a finished request's context (and with it its results) out of the pool until the next
    // run starts: a run of no more requests than contexts then leaves every request's output in a context of its own
    bool recycle_contexts = true;
    void release_ctx(ReqCtx* c) {
        if (!recycle_contexts) { _held.push_back(c); return; }
        { std::lock_guard<std::mutex> lk(_pool_mutex); _pool.push_back(c); }
        _pool_cv.notify_one();
    }

    // ---- profile  (schedule.h:79-157) -----------------------------------------------------------------------
    float lookup(int name, int bs, int seq) {
        auto it = profiling_res_dict.find({name, bs, seq});
        if (it != profiling_res_dict.end()) return it->second;
        if (seq_bucket > 1) {
            it = profiling_res_dict.find({name, bs, (seq + seq_bucket - 1) / seq_bucket * seq_bucket});
            if (it != profiling_res_dict.end()) return it->second;
        }
        profile_misses++;
        return 0.f;  // the reference's operator[] yields 0 for a missing key as well
    }

    // duration of decode-step entry `name` for `bs` token rows at `past` cached positions: the profiled batch at or below bs
    // that exists (a step is weight-streaming bound: its time moves little with the number of rows)
    float lookup_decode(int name, int bs, int past) {
        const int key_past = seq_bucket > 1 ? (past + seq_bucket - 1) / seq_bucket * seq_bucket : past;
        for (int b = bs; b >= 1; --b) {
            auto it = profiling_res_dict.find({name, b, key_past});
            if (it == profiling_res_dict.end()) it = profiling_res_dict.find({name, b, past});
            if (it != profiling_res_dict.end()) return it->second;
        }
        profile_misses++;
        return 0.f;
    }

    void profile_vector(std::vector<FuncWrap>& vec, int count, int name_base, int bs, int key_seq, int itr) {
        void *e0 = nullptr, *e1 = nullptr;
        note_status(lg_event_create(&e0), "lg_event_create");
        note_status(lg_event_create(&e1), "lg_event_create");
        for (int k = 0; k < count; k++) {
            kernel_info info = {name_base + k, bs, key_seq};
            profiling_res_dict[info] = profile_callback(vec[k], DParams0, e0, e1, itr, 3);
            if (vec[k].type == GEMM && vec[k].args_gemm.valid && BertParams.factor > 1) {
                std::vector<float> tmp;
                for (int n = 1; n < BertParams.factor; n++) {
                    FuncWrap fc = decompose_callback(vec[k], BertParams.factor, n, 0.f, 0, axis);
                    tmp.push_back(profile_callback(fc, DParams0, e0, e1, itr, 3));
                }
                profiling_decompse_res_dict[info] = tmp;
            }
        }
        lg_event_destroy(e0);
        lg_event_destroy(e1);
    }

    // Profiles every (bs, seq) in the given ranges with bs*seq % 4 == 0, like the reference; seq advances by seq_step.
    void profile(int low_bs, int high_bs, int low_sq, int high_sq, const std::string& main_filename,
                 const std::string& sub_filename, int seq_step = 1, int itr = 20) {
        for (int i = low_bs; i < high_bs; i++) {
            for (int j = low_sq; j < high_sq; j += seq_step) {
                if ((i * j) % 4 != 0) continue;
                std::vector<FuncWrap> vec = _model->forward(input, output, i, j);
                // run the layer once so that every kernel is timed on initialised data
                for (int k = 0; k < BertParams.kernel_num; k++) vec[k].callback(DParams0);
                profile_vector(vec, BertParams.kernel_num, 0, i, j, itr);
            }
        }
        if (SParams.world_rank == 0) {
            if (!main_filename.empty()) MainDictToFile(profiling_res_dict, main_filename);
            if (!sub_filename.empty()) SubDictToFile(profiling_decompse_res_dict, sub_filename);
        }
    }
    // Profiles one decode step at `past` cached positions; keys are {1000 + k, bs, past}.
    void profile_decode(int bs, int past, int itr = 20) {
        if (bs > BertParams.max_batch_size || BertParams.max_cache_len <= 0 || past < 0 || past >= BertParams.max_cache_len) {
            if (error_code() == 0) set_error_state(LG_ERR_INVALID, "profile_decode: batch or cached positions exceed the model's KV cache");
            return;
        }
        std::vector<FuncWrap> vec = _model->forward_decode(input, output, bs, past, 0);
        const int count = _model->kernels_per_layer(true);
        for (int k = 0; k < count; k++) vec[k].callback(DParams0);
        profile_vector(vec, count, 1000, bs, past, itr);
    }

    // ---- contention ----------------------------------------------------------------------------------------------------
    float contention(int main_class, int sub_class) const {
        if (policy == RESOURCE && main_class >= 0 && main_class < 3 && sub_class >= 0 && sub_class < 3 &&
            contention_table[main_class][sub_class] >= 0.f)
            return contention_table[main_class][sub_class];
        return contention_factor;
    }
    struct ContentionSample { float main_ms, sub_ms, both_ms, hidden; int sub_repeats; };
    // Measures how much of a decode step (HBM-bound kernels, `dec_bs` sequences with `past` cached positions) is hidden
    // when it runs on stream 1 next to the MFMA-bound kernels of one prefill layer (bs x seq) on stream 0, and fills
    // contention_table[MFMA_BOUND][HBM_BOUND] and [HBM_BOUND][MFMA_BOUND].  The decode step is repeated so that both
    // sides are about equally long.  Needs one pool context (the decode side uses its workspace and cache slot).
    ContentionSample profile_contention(int bs, int seq, int dec_bs, int past, int trials = 3) {
        ContentionSample r = {0.f, 0.f, 0.f, -1.f, 0};
        if (_all_ctx.empty() || BertParams.max_cache_len <= 0) return r;
        if (bs <= 0 || seq <= 0 || bs > BertParams.max_batch_size || seq > BertParams.max_seq_len || dec_bs <= 0 || dec_bs > _ctx_batch ||
            past < 0 || past >= BertParams.max_cache_len) return r;
        ReqCtx* c = _all_ctx[0];
        std::vector<FuncWrap> pre = _model->forward(input, output, bs, seq);
        std::vector<FuncWrap> A;
        for (int k = 0; k < BertParams.kernel_num; k++)
            if (pre[k].rclass == MFMA_BOUND) A.push_back(pre[k]);
        const int kd = _model->kernels_per_layer(true);
        std::vector<FuncWrap> dec = _model->forward_decode(c->dec_a, c->dec_b, dec_bs, past, c->slot, c->ws);
        std::vector<FuncWrap> B(dec.begin(), dec.begin() + kd);
        if (A.empty() || B.empty()) return r;
        void *e0 = nullptr, *eA = nullptr, *eB = nullptr;
        note_status(lg_event_create(&e0), "lg_event_create");
        note_status(lg_event_create(&eA), "lg_event_create");
        note_status(lg_event_create(&eB), "lg_event_create");
        // one prefill pass first: every kernel then runs on initialised data
        for (int k = 0; k < BertParams.kernel_num; k++) pre[k].callback(DParams0);
        // returns {time of stream 0's part, time of stream 1's part} of one concurrent run, both from a common start
        auto run = [&](int nA, int nB, float& tA, float& tB) {
            note_status(lg_device_synchronize(), "lg_device_synchronize");
            note_status(lg_event_record(e0, DParams0.stream), "lg_event_record");
            note_status(lg_stream_wait_event(DParams1.stream, e0), "lg_stream_wait_event");
            for (int i = 0; i < nA; ++i) for (auto& f : A) f.callback(DParams0);
            for (int i = 0; i < nB; ++i) for (auto& f : B) f.callback(DParams1);
            note_status(lg_event_record(eA, DParams0.stream), "lg_event_record");
            note_status(lg_event_record(eB, DParams1.stream), "lg_event_record");
            note_status(lg_event_synchronize(eA), "lg_event_synchronize");
            note_status(lg_event_synchronize(eB), "lg_event_synchronize");
            note_status(lg_event_elapsed_ms(&tA, e0, eA), "lg_event_elapsed_ms");
            note_status(lg_event_elapsed_ms(&tB, e0, eB), "lg_event_elapsed_ms");
        };
        float a, b, best_main = 1e30f, best_one = 1e30f;
        run(1, 1, a, b);  // warm-up of both sides
        for (int t = 0; t < trials; ++t) { run(1, 0, a, b); best_main = std::min(best_main, a); }
        for (int t = 0; t < trials; ++t) { run(0, 1, a, b); best_one = std::min(best_one, b); }
        const int reps = std::max(1, (int)(best_main / std::max(best_one, 1e-6f) + 0.5f));
        float best_sub = 1e30f, best_both = 1e30f;
        for (int t = 0; t < trials; ++t) { run(0, reps, a, b); best_sub = std::min(best_sub, b); }
        for (int t = 0; t < trials; ++t) { run(1, reps, a, b); best_both = std::min(best_both, std::max(a, b)); }
        lg_event_destroy(e0); lg_event_destroy(eA); lg_event_destroy(eB);
        const float hidden_ms = best_main + best_sub - best_both;
        auto clamp = [](float x) { return x < 0.05f ? 0.05f : (x > 1.f ? 1.f : x); };
        r.main_ms = best_main; r.sub_ms = best_sub; r.both_ms = best_both; r.sub_repeats = reps;
        r.hidden = clamp(hidden_ms / best_sub);
        contention_table[MFMA_BOUND][HBM_BOUND] = r.hidden;
        contention_table[HBM_BOUND][MFMA_BOUND] = clamp(hidden_ms / best_main);
        return r;
    }

    struct PartitionSample { float main_ms, sub_ms, main_part_ms, sub_part_ms, factor, gain; int sub_repeats; };
    // Measures a partitioned co-run: the MFMA-bound kernels of one prefill layer (bs x seq) on the MFMA side's compute units
    // next to `reps` decode steps (dec_bs sequences, `past` cached positions) on the HBM side's, against both run one after the
    // other on the whole chip.  factor = stand-alone ms of decode work completed per stand-alone ms of prefill work while both
    // run; gain = whole-chip back-to-back time / partitioned co-run time of the same work.  Fills partition_table (both
    // directions) when gain exceeds min_gain, clears it otherwise.  Needs enable_partition, a pool context and a KV cache.
    PartitionSample profile_partition(int bs, int seq, int dec_bs, int past, int trials = 3, float min_gain = 1.02f) {
        PartitionSample r = {0.f, 0.f, 0.f, 0.f, -1.f, 0.f, 0};
        if (partition_hbm_cus <= 0 || _all_ctx.empty() || BertParams.max_cache_len <= 0) return r;
        if (bs <= 0 || seq <= 0 || bs > BertParams.max_batch_size || seq > BertParams.max_seq_len || dec_bs <= 0 || dec_bs > _ctx_batch ||
            past < 0 || past >= BertParams.max_cache_len) return r;
        ReqCtx* c = _all_ctx[0];
        std::vector<FuncWrap> pre = _model->forward(input, output, bs, seq);
        std::vector<FuncWrap> A;
        for (int k = 0; k < BertParams.kernel_num; k++)
            if (pre[k].rclass == MFMA_BOUND) A.push_back(pre[k]);
        const int kd = _model->kernels_per_layer(true);
        std::vector<FuncWrap> dec = _model->forward_decode(c->dec_a, c->dec_b, dec_bs, past, c->slot, c->ws);
        std::vector<FuncWrap> B(dec.begin(), dec.begin() + kd);
        if (A.empty() || B.empty()) return r;
        void *e0 = nullptr, *eA = nullptr, *eB = nullptr;
        note_status(lg_event_create(&e0), "lg_event_create");
        note_status(lg_event_create(&eA), "lg_event_create");
        note_status(lg_event_create(&eB), "lg_event_create");
        for (int k = 0; k < BertParams.kernel_num; k++) pre[k].callback(DParams0);
        auto run = [&](const DynamicInitParam& DA, const DynamicInitParam& DB, int nA, int nB, float& tA, float& tB) {
            note_status(lg_device_synchronize(), "lg_device_synchronize");
            note_status(lg_event_record(e0, DA.stream), "lg_event_record");
            note_status(lg_stream_wait_event(DB.stream, e0), "lg_stream_wait_event");
            for (int i = 0; i < nA; ++i) for (auto& f : A) f.callback(DA);
            for (int i = 0; i < nB; ++i) for (auto& f : B) f.callback(DB);
            note_status(lg_event_record(eA, DA.stream), "lg_event_record");
            note_status(lg_event_record(eB, DB.stream), "lg_event_record");
            note_status(lg_event_synchronize(eA), "lg_event_synchronize");
            note_status(lg_event_synchronize(eB), "lg_event_synchronize");
            note_status(lg_event_elapsed_ms(&tA, e0, eA), "lg_event_elapsed_ms");
            note_status(lg_event_elapsed_ms(&tB, e0, eB), "lg_event_elapsed_ms");
        };
        const DynamicInitParam& PM = *_part[0][MFMA_BOUND];
        const DynamicInitParam& SH = *_part[1][HBM_BOUND];
        float a, b, main_full = 1e30f, sub_full = 1e30f;
        run(DParams0, DParams1, 1, 1, a, b);  // warm-up on the whole chip and on the shares
        run(PM, SH, 1, 1, a, b);
        for (int t = 0; t < trials; ++t) { run(DParams0, DParams1, 1, 0, a, b); main_full = std::min(main_full, a); }
        for (int t = 0; t < trials; ++t) { run(DParams0, DParams1, 0, 1, a, b); sub_full = std::min(sub_full, b); }
        // as many decode steps as finish together with the prefill kernels: start from the whole-chip ratio, correct once
        int reps = std::max(1, (int)(main_full / std::max(sub_full, 1e-6f) + 0.5f));
        float best_a = 0.f, best_b = 0.f;
        for (int pass = 0; pass < 2; ++pass) {
            float best = 1e30f;
            for (int t = 0; t < trials; ++t) {
                run(PM, SH, 1, reps, a, b);
                if (std::max(a, b) < best) { best = std::max(a, b); best_a = a; best_b = b; }
            }
            if (pass == 0) {
                const int adj = std::max(1, (int)((float)reps * best_a / std::max(best_b, 1e-6f) + 0.5f));
                if (adj == reps) break;
                reps = adj;
            }
        }
        lg_event_destroy(e0); lg_event_destroy(eA); lg_event_destroy(eB);
        r.main_ms = main_full; r.sub_ms = sub_full; r.main_part_ms = best_a; r.sub_part_ms = best_b; r.sub_repeats = reps;
        // decode work per millisecond of co-run, times how long the prefill kernels take there, per millisecond of their own
        r.factor = ((float)reps * sub_full / std::max(best_b, 1e-6f)) * best_a / std::max(main_full, 1e-6f);
        r.gain = (main_full + (float)reps * sub_full) / std::max(std::max(best_a, best_b), 1e-6f);
        if (r.gain >= min_gain && r.factor > 0.f && partition_streams_concurrent != 0) {
            partition_table[MFMA_BOUND][HBM_BOUND] = r.factor;
            partition_table[HBM_BOUND][MFMA_BOUND] = 1.0f / r.factor;
        } else {
            partition_table[MFMA_BOUND][HBM_BOUND] = partition_table[HBM_BOUND][MFMA_BOUND] = -1.f;
        }
        return r;
    }

    // ---- serve  (schedule.h:159-172) ------------------------------------------------------------------------
    // Builds the launch vector of one request (prefill of batch_size x seq_len, then n_decode decode steps), stamps
    // kernel indices and profiled durations, and queues it.
    bool serve(int batch_size, int seq_len, int n_decode = 0) {
        if (!request_fits(batch_size, seq_len, n_decode, "serve")) return false;
        ReqCtx* ctx = _pool_total ? acquire_ctx() : nullptr;  // without a pool all requests share the default buffers
        if (_pool_total && !ctx) {
            if (error_code() == 0) set_error_state(LG_ERR_INVALID, "serve: every request context is in flight and no scheduler loop is running to return one");
            return false;
        }
        T* in = ctx ? ctx->input : input;
        T* out = ctx ? ctx->output : output;
        T* ws = ctx ? ctx->ws : nullptr;
        const int slot = (ctx && BertParams.max_cache_len > 0) ? ctx->slot : -1;
        std::unique_lock<std::mutex> build_lock(_build_mutex);  // the layer classes keep per-call state: one builder at a time
        const bool defer_decode = batch_decode && n_decode > 0 && ctx && slot >= 0;  // the decode steps join the batched launch vector
        const bool chunked = defer_decode && prefill_chunk > 0 && batch_size == 1 && seq_len > prefill_chunk && BertParams.fused;
        std::vector<FuncWrap> vec;
        int key_len = seq_len;
        if (chunked) {
            const int H = BertParams.head_num * BertParams.size_per_head;
            for (int p0 = 0; p0 < seq_len; p0 += prefill_chunk) {
                const int c = std::min(prefill_chunk, seq_len - p0);
                std::vector<FuncWrap> cv = _model->forward_prefill_past(in + (int64_t)p0 * H, out + (int64_t)p0 * H, 1, c, p0, ws, slot);
                for (size_t j = 0; j < cv.size(); ++j) {
                    cv[j].name = (int)(j % (size_t)BertParams.kernel_num);
                    cv[j].duration = lookup(cv[j].name, 1, c);
                }
                if (p0 + c < seq_len && !cv.empty()) cv.back().yield_after = true;
                vec.insert(vec.end(), cv.begin(), cv.end());
            }
            key_len = prefill_chunk;
        } else {
            vec = _model->forward(in, out, batch_size, seq_len, ws, slot);
            for (int i = 0; i < BertParams.layer_num; i++)
                for (int j = 0; j < BertParams.kernel_num; j++) {
                    FuncWrap& f = vec[i * BertParams.kernel_num + j];
                    f.name = j;
                    f.duration = lookup(j, batch_size, seq_len);
                }
        }
        if (n_decode > 0 && ctx && slot >= 0 && !defer_decode) {
            const int H = BertParams.head_num * BertParams.size_per_head;
            const int kd = _model->kernels_per_layer(true);
            T* din = ctx->dec_a;
            T* dout = ctx->dec_b;
            // the last token's hidden state of every sequence becomes the first decode input
            {
                const size_t row_bytes = (size_t)H * sizeof(T);
                FuncWrap g(0.01f, COMPUTATION, [=](const DynamicInitParam& D) {
                    for (int b = 0; b < batch_size; ++b)
                        note_status(lg_memcpy_d2d_async((char*)din + b * row_bytes,
                                                        (const char*)out + ((size_t)(b + 1) * seq_len - 1) * row_bytes, row_bytes,
                                                        D.stream), "lg_memcpy_d2d_async");
                }, "gather_last_token");
                g.minor = true;
                g.name = 900;
                g.duration = 0.005f;
                vec.push_back(g);
            }
            for (int t = 0; t < n_decode; ++t) {
                const int past = seq_len + t;
                std::vector<FuncWrap> dv = _model->forward_decode(din, dout, batch_size, past, slot, ws);
                const int key_past = seq_bucket > 1 ? (past + seq_bucket - 1) / seq_bucket * seq_bucket : past;
                for (size_t j = 0; j < dv.size(); ++j) {
                    dv[j].name = 1000 + (int)(j % kd);
                    dv[j].duration = lookup(dv[j].name, batch_size, key_past);
                }
                vec.insert(vec.end(), dv.begin(), dv.end());
                std::swap(din, dout);
            }
        }
        build_lock.unlock();
        Sample* sample = new Sample(vec, profiling_decompse_res_dict, batch_size, seq_len, BertParams.factor, policy, axis);
        sample->user = ctx;
        sample->merge_minor = merge_minor;
        sample->key_seq = seq_bucket > 1 ? (key_len + seq_bucket - 1) / seq_bucket * seq_bucket : key_len;  // chunks: a chunk's GEMMs are what gets split
        sample->n_decode_pending = defer_decode ? n_decode : 0;
        sample->chunked = chunked;
        {
            std::lock_guard<std::mutex> lk(_q_mutex);
            sample->id = _next_id++;
            _main_q.push_back(sample);
        }
        return true;
    }

    // Queues a request that consists of decode steps only: `n_steps` single-token steps for `batch_size` sequences that
    // already have `past` cached positions (cache contents are whatever the slot holds).  No reference counterpart.
    bool serve_decode(int batch_size, int past, int n_steps) {
        if (!decode_fits(batch_size, past, n_steps, "serve_decode")) return false;
        ReqCtx* ctx = _pool_total ? acquire_ctx() : nullptr;
        if (_pool_total && !ctx) {
            if (error_code() == 0) set_error_state(LG_ERR_INVALID, "serve_decode: every request context is in flight and no scheduler loop is running to return one");
            return false;
        }
        T* din = ctx ? ctx->dec_a : input;
        T* dout = ctx ? ctx->dec_b : output;
        T* ws = ctx ? ctx->ws : nullptr;
        const int slot = ctx ? ctx->slot : 0;
        const int kd = _model->kernels_per_layer(true);
        std::unique_lock<std::mutex> build_lock(_build_mutex);
        std::vector<FuncWrap> vec;
        for (int t = 0; t < n_steps; ++t) {
            const int p = past + t;
            std::vector<FuncWrap> dv = _model->forward_decode(din, dout, batch_size, p, slot, ws);
            const int key_past = seq_bucket > 1 ? (p + seq_bucket - 1) / seq_bucket * seq_bucket : p;
            for (size_t j = 0; j < dv.size(); ++j) {
                dv[j].name = 1000 + (int)(j % kd);
                dv[j].duration = lookup(dv[j].name, batch_size, key_past);
            }
            vec.insert(vec.end(), dv.begin(), dv.end());
            std::swap(din, dout);
        }
        build_lock.unlock();
        Sample* sample = new Sample(vec, profiling_decompse_res_dict, batch_size, past, BertParams.factor, policy, axis);
        sample->user = ctx;
        sample->merge_minor = merge_minor;
        {
            std::lock_guard<std::mutex> lk(_q_mutex);
            sample->id = _next_id++;
            _main_q.push_back(sample);
        }
        return true;
    }

    size_t queued() {
        std::lock_guard<std::mutex> lk(_q_mutex);
        return _main_q.size();
    }

    // ---- admission / retirement  (schedule.h:175-202) ------------------------------------------------------------
    void update_vec() {
        if (batch_decode) _update_decode_batch();
        if (!exe_vec.empty() && exe_vec[0] != _dec_sample && exe_vec[0]->empty()) {
            Sample* tmp = exe_vec[0];
            recs.push_back(tmp->get_recording());
            sub_profile_misses += tmp->sub_profile_misses;
            exe_vec.erase(exe_vec.begin());
            _retired.push_back(tmp);
        }
        _reclaim();
        const size_t deep = (size_t)schedule_deep + (_dec_sample ? 1 : 0);  // the batched step does not use up a request's place
        for (size_t i = exe_vec.size(); i < deep; i++) {
            std::lock_guard<std::mutex> lk(_q_mutex);
            if (_main_q.empty()) break;
            // the batched decode step stays last: a request's prefill goes ahead of it (the request then joins the batch)
            exe_vec.insert(_dec_sample ? exe_vec.end() - 1 : exe_vec.end(), _main_q.front());
            if (_main_q.front()->chunked) chunked_prefills++;
            _main_q.pop_front();
        }
        if (exe_vec.empty()) std::this_thread::sleep_for(std::chrono::microseconds(100));
    }

    bool drained() { return exe_vec.empty() && queued() == 0 && _dec_seqs.empty(); }

    // ---- baseline: one request at a time on stream 0  (schedule.h:204-219) -----------------------------------------
    void run_sequential() {
        RunningGuard running(this);
        float time_planned = 0;
        note_status(lg_event_record(Wait_EVENT, DParams0.stream), "lg_event_record");
        while (!(_stop.load() && drained())) {
            update_vec();
            if (!exe_vec.empty()) {
                note_status(lg_event_synchronize(Wait_EVENT), "lg_event_synchronize");
                // one request at a time, to its end -- or to the end of a chunk of a chunked prefill, after which the batched
                // decode step (if there is one) has its turn before the next chunk
                Sample* cur = _pick_head();
                bool yielded = false;
                while (!cur->empty() && !yielded) {
                    yielded = cur->next_yields();
                    cur->dequeue(DParams0, 1, time_planned);
                }
                _yield_turn = yielded;
                note_status(lg_event_record(Wait_EVENT, DParams0.stream), "lg_event_record");
                rounds++;
            }
        }
        _finish();
    }

    // ---- Liger: interleave the waiting requests into the primary's windows  (schedule.h:221-278) ----------------------
    void run_stream_sync() {
        RunningGuard running(this);
        // two requests on two streams must not share buffers: without per-request contexts only one request may be in flight
        if (_pool_total == 0 && schedule_deep > 1) {
            if (error_code() == 0) set_error_state(LG_ERR_INVALID, "run_stream_sync: interleaving needs per-request contexts (make_pool) or schedule_deep 1");
            _drop_queued();
            return;
        }
        float time_planned = 0.0f;
        int main_class = 0;
        note_status(lg_event_record(Wait_EVENT, DParams0.stream), "lg_event_record");
        note_status(lg_event_record(Main_EVENT, DParams0.stream), "lg_event_record");
        while (!(_stop.load() && drained())) {
            update_vec();
            if (exe_vec.empty()) continue;
            Sample* head = _pick_head();
            // Partitioned round?  Only while a waiting request has work of the other class at its head, and only for as much
            // primary time as that work needs; the primary then runs on its class's share of the compute units, the
            // secondaries on the other share.  Otherwise (and always without enable_partition) the round is the reference's:
            // primary on stream 0, secondaries on stream 1, both on the whole chip.
            const DynamicInitParam* Dp = &DParams0;
            const DynamicInitParam* Ds = &DParams1;
            float part_factor = -1.f, cap = 0.f;
            int round_kind = 0;   // 0: no partition possible, 1: possible but run on the whole chip, 2: partitioned
            if (partition_hbm_cus > 0 && policy == RESOURCE && !head->empty()) {
                const int mc = head->next_class();
                const int sc = mc == MFMA_BOUND ? HBM_BOUND : (mc == HBM_BOUND ? MFMA_BOUND : -1);
                if (sc >= 0 && partition_table[mc][sc] > 0.f) {
                    float need = 0.f;
                    for (Sample* other : exe_vec)
                        if (other != head && !other->empty()) need += other->run_ahead_duration(mc);
                    if (need >= partition_min_ms) {
                        round_kind = _partition_pays() ? 2 : 1;
                        if (round_kind == 2) {
                            part_factor = partition_table[mc][sc];
                            cap = need / part_factor;
                            Dp = _part[0][mc];
                            Ds = _part[1][sc];
                            partition_rounds++;
                        } else {
                            partition_declined++;
                        }
                    }
                }
            }
            // hybrid synchronisation: the host waits for everything before the last kernel of the previous round,
            // the secondary stream waits (on the device) for the end of the previous round
            note_status(lg_event_synchronize(Wait_EVENT), "lg_event_synchronize");
            note_status(lg_stream_wait_event(Ds->stream, Main_EVENT), "lg_stream_wait_event");
            if (partition_feedback && partition_hbm_cus > 0) _round_begin(*Dp, round_kind);
            float round_work = 0.f;
            while (!head->empty()) {
                main_class = head->next_class();
                const bool capped = part_factor > 0.f && time_planned + head->duration(1, time_planned) >= cap;
                if (head->is_switch() || capped) {
                    _yield_turn = head->next_yields();
                    note_status(lg_event_record(Wait_EVENT, Dp->stream), "lg_event_record");
                    time_planned += head->dequeue(*Dp, 1, time_planned);
                    note_status(lg_event_record(Main_EVENT, Dp->stream), "lg_event_record");
                    break;
                }
                time_planned += head->dequeue(*Dp, 1, time_planned);
            }
            round_work += time_planned;
            rounds++;
            // time_planned stays in units of the primary's time; a secondary kernel of stand-alone duration d uses up
            // d / contention(main, sub) of it (with the constant factor this is the reference's 0.8 x time_planned budget)
            for (Sample* sub : exe_vec) {
                if (sub == head) continue;
                while (time_planned > 0 && !sub->empty()) {
                    if (sub->is_same_class(main_class)) break;
                    const float f = part_factor > 0.f ? part_factor : contention(main_class, sub->next_class());
                    float avail = time_planned * f;
                    if (sub->duration(0, avail) > avail) {
                        if (sub->type() == GEMM && sub->possible_duration(avail)) {
                            splits++;
                            continue;  // the first piece now fits
                        }
                        time_planned = 0.0f;
                    } else {
                        const float d = sub->dequeue(*Ds, 0, avail);
                        time_planned -= d / f;
                        round_work += d;
                        secondary_launches++;
                    }
                }
            }
            time_planned = 0.0f;
            if (!_round_log.empty()) _round_log.back().work = round_work;
        }
        _finish();
    }

    void run_stop() { _stop.store(true); }
    void reset_run() {
        _stop.store(false);
        if (!_held.empty()) {
            { std::lock_guard<std::mutex> lk(_pool_mutex); for (ReqCtx* c : _held) _pool.push_back(c); }
            _held.clear();
            _pool_cv.notify_all();
        }
        // epoch of the run: an event whose host time is known (the stream is idle, so it completes as it is recorded)
        if (!_epoch_event) note_status(lg_event_create(&_epoch_event), "lg_event_create");
        note_status(lg_stream_synchronize(DParams0.stream), "lg_stream_synchronize");
        note_status(lg_event_record(_epoch_event, DParams0.stream), "lg_event_record");
        note_status(lg_event_synchronize(_epoch_event), "lg_event_synchronize");
        _epoch_host = std::chrono::steady_clock::now();
        for (auto& r : recs) { lg_event_destroy(r.start); lg_event_destroy(r.stop); }
        recs.clear();
        for (void* e : _dec_prefill_events) lg_event_destroy(e);
        _dec_prefill_events.clear();
        if (_dec_prev_stop) { lg_event_destroy(_dec_prev_stop); _dec_prev_stop = nullptr; }
        batched_steps = batched_rows = 0;
        rounds = secondary_launches = splits = partition_rounds = partition_declined = 0;
        chunked_prefills = yield_turns = 0;
        _yield_turn = false;
        // what the rounds of earlier runs delivered is kept (it is a property of the device and the workload, and a run may have
        // few rounds in which a partition is possible); older samples count half at every new run
        for (RoundRec& r : _round_log) _round_events.push_back(r.begin);
        _round_log.clear();
        for (int k = 0; k < 3; ++k) { _fb_work[k] *= 0.5; _fb_time[k] *= 0.5; }
    }

    // ---- request simulator  (schedule.h:285-321) ---------------------------------------------------------------------
    // Replays `trace` in real time on a second host thread, then requests stop.
    void serving(const std::vector<TraceRequest>& trace) {
        if (_thread.joinable()) _thread.join();
        _running.store(true);  // a loop is about to run: serve() may wait for a context instead of failing
        _thread = std::thread([this, trace]() {
            const auto t0 = std::chrono::steady_clock::now();
            for (const auto& r : trace) {
                std::this_thread::sleep_until(t0 + std::chrono::duration_cast<std::chrono::steady_clock::duration>(
                                                       std::chrono::duration<double>(r.arrival_s)));
                serve(r.batch, r.seq, r.n_decode);
            }
            run_stop();
        });
    }
    // the reference's generator: `count` requests of max batch, seq = rand() % (max_seq_len - 28) + 16 accepted when
    // batch*seq % 4 == 0, spaced by rq_interval microseconds
    std::vector<TraceRequest> reference_trace(int count, unsigned seed = 1) {
        std::vector<TraceRequest> tr;
        srand(seed);
        double t = 0;
        while ((int)tr.size() < count) {
            const int bs = BertParams.max_batch_size;
            const int sq = (rand() % (BertParams.max_seq_len - 28)) + 16;
            if ((bs * sq) % 4 == 0) {
                tr.push_back({t, bs, sq, 0});
                t += BertParams.rq_interval * 1e-6;
            }
        }
        return tr;
    }

    // ---- report  (schedule.h:325-350) ----------------------------------------------------------------------------------
    Report output_recording(bool print = true) {
        std::vector<double> cpu, gpu;
        const size_t skip = std::min((size_t)std::max(0, ignore_num), recs.size());
        for (size_t i = skip; i < recs.size(); ++i) {
            float ms = 0.f;
            note_status(lg_event_elapsed_ms(&ms, recs[i].start, recs[i].stop), "lg_event_elapsed_ms");
            cpu.push_back(recs[i].cpu_time * 1000.0);
            gpu.push_back(ms);
            if (print) printf("request: %zu, CPU_Time: %f ms, CUDA_Time: %f ms. \n", i - skip, cpu.back(), gpu.back());
        }
        // first start -> last stop (schedule.h:340-343 takes the last record's stop; a request that ran on the second stream may
        // finish before the one retired ahead of it, so the latest stop is looked for)
        float total = 0.f;
        for (size_t i = skip; i < recs.size(); ++i) {
            float ms = 0.f;
            note_status(lg_event_elapsed_ms(&ms, recs[skip].start, recs[i].stop), "lg_event_elapsed_ms");
            total = std::max(total, ms);
        }
        Report r = summarize_records(cpu, gpu, total);
        if (_epoch_event && recs.size() > skip) {
            std::vector<double> e2e;
            for (size_t i = skip; i < recs.size(); ++i) {
                float done = 0.f;
                note_status(lg_event_elapsed_ms(&done, _epoch_event, recs[i].stop), "lg_event_elapsed_ms");
                e2e.push_back((double)done - std::chrono::duration<double, std::milli>(recs[i].arrive - _epoch_host).count());
            }
            double sum = 0;
            for (double v : e2e) sum += v;
            r.avg_e2e_ms = sum / (double)e2e.size();
            std::sort(e2e.begin(), e2e.end());
            size_t rank = (size_t)std::ceil(0.99 * (double)e2e.size());
            r.p99_e2e_ms = e2e[std::min(e2e.size() - 1, rank ? rank - 1 : 0)];
        }
        if (print) {
            printf("Total_Duration: %f ms. \n", r.total_duration_ms);
            printf("Throughput: %f samples/s. \n", r.throughput);
            printf("Average Latency: %f ms. \n", r.avg_latency_ms);
            printf("P99 Latency: %f ms. \n", r.p99_latency_ms);
            printf("Total %d records. \n", r.records);
        }
        return r;
    }

  private:
    // ---- batched decode steps ---------------------------------------------------------------------------------------------
    struct DecodeSeq {
        ReqCtx* ctx;
        int batch, seq_len, past, remaining, n_decode;
        bool joined;
        void *start, *prefill_done, *done;   // events: first prefill kernel, last prefill kernel, last decode kernel
        double cpu_time;
        std::chrono::steady_clock::time_point arrive;
    };
    std::vector<DecodeSeq> _dec_seqs;        // requests in (or about to join) their decode steps
    Sample* _dec_sample = nullptr;           // launch vector of the batched step(s) being launched; last in exe_vec while it exists
    T *_dec_x = nullptr, *_dec_ws = nullptr; // token rows [contexts x ctx_batch, hidden] (a step runs in place) and its workspace
    std::vector<std::pair<void*, ReqCtx*>> _dec_done;   // (completion event, context to hand back)
    std::mutex _build_mutex;

    // requests whose prefill vector has been launched completely move on to the decode batch
    void _collect_prefilled() {
        for (size_t i = 0; i < exe_vec.size();) {
            Sample* smp = exe_vec[i];
            if (smp == _dec_sample || !smp->empty() || smp->n_decode_pending <= 0) { ++i; continue; }
            DecodeSeq q;
            q.ctx = (ReqCtx*)smp->user;
            q.batch = smp->batch_size; q.seq_len = smp->seq_len; q.past = smp->seq_len;
            q.remaining = q.n_decode = smp->n_decode_pending;
            q.joined = false;
            q.start = smp->start; q.prefill_done = smp->stop; q.done = nullptr;
            note_status(lg_event_create(&q.done), "lg_event_create");
            q.cpu_time = smp->time_cpu_elapsed();
            q.arrive = smp->sample_arrive;
            sub_profile_misses += smp->sub_profile_misses;
            _dec_seqs.push_back(q);
            exe_vec.erase(exe_vec.begin() + i);
            delete smp;
        }
    }

    // Builds the launch vector of the next batched step(s): [join] step [retire] step [retire] ...
    //   join:   every request that has finished its prefill since the last vector waits (on the device) for its last prefill
    //           kernel and copies the hidden state of its last token into its row of the batch;
    //   step:   one decode step over rows 0 .. highest row in use (rows of no request point at the spare cache slot);
    //   retire: requests that have run their last step copy their row out and record their completion event.
    void _build_decode_vector() {
        const int H = BertParams.head_num * BertParams.size_per_head;
        const size_t row_bytes = (size_t)H * sizeof(T);
        const int kd = _model->kernels_per_layer(true);
        const int spare_slot = _pool_total * _ctx_batch;
        bool waiting = queued() > 0;
        for (Sample* smp : exe_vec) waiting = waiting || smp != _dec_sample;
        int steps = 1;
        if (!waiting) {
            steps = 0;
            for (const DecodeSeq& q : _dec_seqs) steps = std::max(steps, q.remaining);
            steps = std::max(1, std::min(steps, decode_steps_ahead));
        }
        std::vector<FuncWrap> vec;
        // join
        {
            std::vector<DecodeSeq*> joiners;
            for (DecodeSeq& q : _dec_seqs)
                if (!q.joined) { joiners.push_back(&q); q.joined = true; }
            if (!joiners.empty()) {
                struct Join { void* done; const char* src; char* dst; int batch, seq_len; };
                std::vector<Join> js;
                for (DecodeSeq* q : joiners)
                    js.push_back({q->prefill_done, (const char*)q->ctx->output, (char*)_dec_x + (size_t)q->ctx->slot * row_bytes, q->batch, q->seq_len});
                FuncWrap f(0.005f, COMPUTATION, [js, row_bytes](const DynamicInitParam& D) {
                    for (const Join& j : js) {
                        note_status(lg_stream_wait_event(D.stream, j.done), "lg_stream_wait_event");
                        for (int b = 0; b < j.batch; ++b)
                            note_status(lg_memcpy_d2d_async(j.dst + (size_t)b * row_bytes, j.src + ((size_t)(b + 1) * j.seq_len - 1) * row_bytes,
                                                            row_bytes, D.stream), "lg_memcpy_d2d_async");
                    }
                }, "join_decode_batch");
                f.minor = true; f.name = 900; f.duration = 0.005f;
                vec.push_back(f);
            }
        }
        // The steps of this vector work in place on the batch's rows, workspace and cache slots, like the steps of the vector
        // before it, whose last kernels may still be running on the other stream: the vector's first entry waits for them.
        if (_dec_prev_stop) {
            void* prev = _dec_prev_stop;
            FuncWrap f(0.001f, COMPUTATION, [prev](const DynamicInitParam& D) {
                note_status(lg_stream_wait_event(D.stream, prev), "lg_stream_wait_event");
            }, "after_previous_steps");
            f.minor = true; f.name = 902; f.duration = 0.001f;
            vec.insert(vec.begin(), f);
        }
        std::unique_lock<std::mutex> build_lock(_build_mutex);
        for (int st = 0; st < steps; ++st) {
            int rows = 0, longest = 0;
            for (const DecodeSeq& q : _dec_seqs)
                if (q.remaining > 0) { rows = std::max(rows, q.ctx->slot + q.batch); longest = std::max(longest, q.past); }
            if (rows == 0) break;
            std::vector<int> slots(rows, spare_slot), pasts(rows, 0);
            for (const DecodeSeq& q : _dec_seqs)
                if (q.remaining > 0)
                    for (int b = 0; b < q.batch; ++b) { slots[q.ctx->slot + b] = q.ctx->slot + b; pasts[q.ctx->slot + b] = q.past; }
            std::vector<FuncWrap> dv = _model->forward_decode_seqs(_dec_x, _dec_x, slots, pasts, _dec_ws);
            for (size_t j = 0; j < dv.size(); ++j) {
                dv[j].name = 1000 + (int)(j % kd);
                dv[j].duration = lookup_decode(dv[j].name, rows, longest);
            }
            vec.insert(vec.end(), dv.begin(), dv.end());
            if (decode_step_hook) {
                const int step_no = batched_steps;
                T* x = _dec_x;
                auto hook = decode_step_hook;
                FuncWrap f(0.001f, COMPUTATION, [hook, step_no, slots, pasts, x](const DynamicInitParam& D) { hook(step_no, slots, pasts, x, D); },
                           "decode_step_hook");
                f.minor = true; f.name = 903; f.duration = 0.001f;
                vec.push_back(f);
            }
            batched_steps++;
            batched_rows += rows;
            // retire
            struct Retire { void* done; const char* src; char* dst; int batch; };
            std::vector<Retire> rs;
            for (DecodeSeq& q : _dec_seqs) {
                if (q.remaining <= 0) continue;
                q.past++;
                if (--q.remaining > 0) continue;
                char* out = (char*)((q.n_decode & 1) ? q.ctx->dec_b : q.ctx->dec_a);   // where the request's own decode steps would leave it
                rs.push_back({q.done, (const char*)_dec_x + (size_t)q.ctx->slot * row_bytes, out, q.batch});
                recs.push_back(recorder{q.cpu_time, q.start, q.done, q.batch, q.seq_len, q.arrive});
                _dec_done.push_back({q.done, q.ctx});
                _dec_prefill_events.push_back(q.prefill_done);
            }
            if (!rs.empty()) {
                FuncWrap f(0.005f, COMPUTATION, [rs, row_bytes](const DynamicInitParam& D) {
                    for (const Retire& r : rs) {
                        note_status(lg_memcpy_d2d_async(r.dst, r.src, (size_t)r.batch * row_bytes, D.stream), "lg_memcpy_d2d_async");
                        note_status(lg_event_record(r.done, D.stream), "lg_event_record");
                    }
                }, "retire_from_decode_batch");
                f.minor = true; f.name = 901; f.duration = 0.005f;
                vec.push_back(f);
            }
            _dec_seqs.erase(std::remove_if(_dec_seqs.begin(), _dec_seqs.end(), [](const DecodeSeq& q) { return q.remaining <= 0; }), _dec_seqs.end());
        }
        build_lock.unlock();
        if (vec.empty()) return;
        _dec_sample = new Sample(vec, profiling_decompse_res_dict, 1, 1, 1, policy, axis);
        _dec_sample->merge_minor = true;   // join / retire entries never end a run
        _dec_sample->id = -1;
        exe_vec.push_back(_dec_sample);
    }

    void _update_decode_batch() {
        _collect_prefilled();
        if (_dec_sample && _dec_sample->empty()) {
            exe_vec.erase(std::find(exe_vec.begin(), exe_vec.end(), _dec_sample));
            lg_event_destroy(_dec_sample->start);
            // the stop event (recorded behind the vector's last kernel) is what the next vector waits for; the one before it
            // is no longer needed: whatever waited for it has been launched, and a wait keeps the state it found at launch
            if (_dec_prev_stop) lg_event_destroy(_dec_prev_stop);
            _dec_prev_stop = _dec_sample->stop;
            delete _dec_sample;
            _dec_sample = nullptr;
        }
        if (!_dec_sample && !_dec_seqs.empty()) _build_decode_vector();
        // contexts of requests whose last decode kernel has finished go back to the pool
        for (size_t i = 0; i < _dec_done.size();) {
            if (lg_event_query(_dec_done[i].first) == LG_OK) {
                release_ctx(_dec_done[i].second);
                _dec_done.erase(_dec_done.begin() + i);
            } else {
                ++i;
            }
        }
    }
    std::vector<void*> _dec_prefill_events;  // destroyed with the run's records
    void* _dec_prev_stop = nullptr;          // stop event of the previous vector of batched steps

    // The primary of the next round: the first request in line -- or, right after a chunk of a chunked prefill, the batched
    // decode step once (if it has launches left), so that the requests in their decode steps advance between two chunks.
    bool _yield_turn = false;
    Sample* _pick_head() {
        Sample* head = exe_vec.at(0);
        if (_yield_turn && _dec_sample && head != _dec_sample && !_dec_sample->empty()) {
            head = _dec_sample;
            yield_turns++;
        }
        _yield_turn = false;
        return head;
    }
    std::atomic<bool> _running{false};
    std::vector<ReqCtx*> _held;   // contexts of finished requests kept back while recycle_contexts is off
    int _ctx_batch = 0;
    struct RunningGuard {
        Scheduler* s;
        explicit RunningGuard(Scheduler* s_) : s(s_) { s->_running.store(true); }
        ~RunningGuard() { s->_running.store(false); s->_pool_cv.notify_all(); }
    };
    void _drop_queued() {
        std::lock_guard<std::mutex> lk(_q_mutex);
        for (Sample* smp : _main_q) delete smp;
        _main_q.clear();
    }
    // ---- partition feedback ------------------------------------------------------------------------------------------------
    struct RoundRec { void* begin; float work; int kind; };
    std::deque<RoundRec> _round_log;     // rounds whose duration is not known yet (the last one is the round being launched)
    std::vector<void*> _round_events;    // pool of events for the log
    double _fb_work[3] = {0, 0, 0}, _fb_time[3] = {0, 0, 0};
    int _fb_n[3] = {0, 0, 0}, _fb_eligible = 0;
    void* _round_event() {
        if (!_round_events.empty()) { void* e = _round_events.back(); _round_events.pop_back(); return e; }
        void* e = nullptr;
        note_status(lg_event_create(&e), "lg_event_create");
        return e;
    }
    // The round's first event: on the primary's stream, behind the end of the primary run before it (Main_EVENT), so that the
    // distance between two such events is the time the earlier round's primary run took, whichever streams the two rounds use.
    // A round's secondary work may still be running then (nothing makes the next primary wait for it) and is then paid for by
    // the round it runs into: the estimate flatters the kind of round whose secondaries run long, which is the partitioned
    // kind (its primary is cut short on purpose).  partition_feedback_margin allows for that.
    void _round_begin(const DynamicInitParam& Dp, int kind) {
        note_status(lg_stream_wait_event(Dp.stream, Main_EVENT), "lg_stream_wait_event");
        RoundRec r{_round_event(), 0.f, kind};
        note_status(lg_event_record(r.begin, Dp.stream), "lg_event_record");
        _round_log.push_back(r);
        // every round but the newest has an end (the next round's beginning): account for those whose events have completed
        while (_round_log.size() >= 2 && lg_event_query(_round_log[1].begin) == LG_OK) {
            RoundRec done = _round_log.front();
            _round_log.pop_front();
            float ms = 0.f;
            if (lg_event_elapsed_ms(&ms, done.begin, _round_log.front().begin) == LG_OK && ms > 0.f && done.kind > 0 && done.work > 0.f) {
                _fb_work[done.kind] += done.work;
                _fb_time[done.kind] += ms;
                _fb_n[done.kind]++;
            }
            _round_events.push_back(done.begin);
        }
    }
    // whether the round that is about to start, in which a partition is possible, should be partitioned
    bool _partition_pays() {
        if (!partition_feedback) return true;
        const int n = _fb_eligible++;
        // both kinds in turn while either lacks samples (launched rounds count: their durations arrive a little later)
        if (_fb_n[1] < partition_feedback_min || _fb_n[2] < partition_feedback_min) return (n & 1) == 0;
        const bool pays = feedback_rate(2) >= (double)partition_feedback_margin * feedback_rate(1);
        if (partition_feedback_probe > 0 && n % partition_feedback_probe == 0) return !pays;
        return pays;
    }
    struct PartStreams { std::unique_ptr<DynamicInitParam> d[2][2]; int verified = -1; };
    static constexpr int PARTITION_STREAM_TRIES = 6;
    // releases every CU-masked stream and leaves partitioning off with no pointer to a released stream behind
    void _drop_partition_streams() {
        partition_hbm_cus = 0;
        for (int role = 0; role < 2; ++role)
            for (int cls = 0; cls < 2; ++cls) _part[role][cls] = nullptr;
        for (auto& kv : _part_streams)
            for (int role = 0; role < 2; ++role)
                for (int cls = 0; cls < 2; ++cls)
                    if (kv.second.d[role][cls]) kv.second.d[role][cls]->destroy();
        _part_streams.clear();
    }
    std::map<int, PartStreams> _part_streams;                              // by HBM-side share, created once
    DynamicInitParam* _part[2][2] = {{nullptr, nullptr}, {nullptr, nullptr}};  // CU-masked streams of partitioned rounds: [role][class]
    void* _epoch_event = nullptr;
    std::chrono::steady_clock::time_point _epoch_host;
    std::vector<Sample*> _retired;
    int _pool_total = 0;
    std::vector<ReqCtx*> _all_ctx;
    // a retired sample's buffers may be reused once its last kernel has finished
    void _reclaim() {
        for (size_t i = 0; i < _retired.size();) {
            Sample* s = _retired[i];
            if (lg_event_query(s->stop) == LG_OK) {
                if (s->user) release_ctx((ReqCtx*)s->user);
                delete s;
                _retired.erase(_retired.begin() + i);
            } else {
                ++i;
            }
        }
    }
    void _finish() {
        note_status(lg_stream_synchronize(DParams0.stream), "lg_stream_synchronize");
        note_status(lg_stream_synchronize(DParams1.stream), "lg_stream_synchronize");
        // every CU-masked stream that exists, whether or not partitioning is switched on at the moment
        for (auto& kv : _part_streams)
            for (int role = 0; role < 2; ++role)
                for (int cls = 0; cls < 2; ++cls)
                    if (kv.second.d[role][cls] && kv.second.d[role][cls]->stream)
                        note_status(lg_stream_synchronize(kv.second.d[role][cls]->stream), "lg_stream_synchronize");
        _reclaim();
        for (auto& d : _dec_done) release_ctx(d.second);   // every stream has been synchronised: their kernels are done
        _dec_done.clear();
        if (_thread.joinable()) _thread.join();
    }
};

}  // namespace liger
