// sample.h -- one in-flight request: its launch vector, a cursor, and the sub-queue of decomposed GEMM pieces.
//
// Counterpart of the reference's src/init.h (Sample, :22-283; recorder :16-20).  Same public surface (dequeue, duration,
// possible_duration, is_switch, is_same_type, type, empty, get_recording ...) and the same policy:
//   * the primary request launches maximal runs of same-class kernels ("rounds"); is_switch() marks the last launch
//     of a run (init.h:121-129);
//   * a secondary request may only co-run kernels of the OTHER class (is_same_type, init.h:131-149);
//   * a GEMM that does not fit the remaining window is split into [largest profiled fraction that fits, remainder]
//     (possible_duration, init.h:226-259) and the remainder can be split again later.
// What "class" means is a policy knob: CLASSIC reproduces the reference (COMMUNICATION vs everything else);
// RESOURCE compares resource classes (MFMA-bound vs HBM-bound), which is what one GPU has to interleave when there is
// no communication entry in the vector.
// Fixes relative to the reference: pieces carry their offset, so the pieces of a GEMM cover its output exactly once
// (the reference re-scales an already scaled problem and always starts at column 0); the remainder keeps its own
// profiled duration (the reference reads vec[1]); a missing profile entry makes possible_duration() return false
// instead of indexing an empty vector; the GPU stop event is recorded after the last launch, so the last kernel
// is inside the measured interval; every launch records a per-sample event so that a request that moves from the
// secondary to the primary stream is ordered after its own earlier kernels.
#pragma once
#include <chrono>

#include "profile_store.h"

namespace liger {

enum class_policy { CLASSIC = 0, RESOURCE = 1 };

struct recorder {     // init.h:16-20
    double cpu_time;  // queueing delay in seconds: first launch - arrival
    void* start;      // events (lg_event_*)
    void* stop;
    int batch_size, seq_len;
    std::chrono::steady_clock::time_point arrive;  // host clock at arrival (not in the reference: end-to-end latency)
};

class Sample {
  private:
    struct Piece {
        FuncWrap func;
        int start, count;  // units [start, start + count) of `_factor`
    };
    std::vector<Piece> _SubFuncWrapVec;
    size_t _sub_exe_num = 0;
    int _factor = 0;
    class_policy _policy = CLASSIC;
    split_axis _axis = SPLIT_OUT_COLS;
    int _last_stream = -1;
    void* _last_stream_handle = nullptr;

    bool _sub_empty() const { return _SubFuncWrapVec.size() == _sub_exe_num; }
    size_t _sub_size() const { return _SubFuncWrapVec.size() - _sub_exe_num; }
    void _sub_clear() { _SubFuncWrapVec.clear(); _sub_exe_num = 0; }
    int _class_of(const FuncWrap& f) const {
        if (_policy == CLASSIC) return f.type == COMMUNICATION ? 0 : 1;
        return (int)f.rclass;
    }
    // RESOURCE policy with merge_minor: a minor entry (FuncWrap::minor) is too small to matter as a resource user and takes the
    // class of the nearest other entry before it (after it, at the head of the vector).  The LayerNorm of a prefill layer (tens
    // of microseconds between milliseconds of GEMMs) then neither ends the primary's run of MFMA-bound launches nor stops a
    // secondary request whose prefill is being interleaved into HBM-bound windows.
    bool _neutral(const FuncWrap& f) const { return _policy == RESOURCE && merge_minor && f.minor && f.type != COMMUNICATION; }
    int _class_at(size_t idx) const {
        const FuncWrap& f = FuncWrapVec.at(idx);
        if (!_neutral(f)) return _class_of(f);
        for (size_t i = idx; i-- > 0;)
            if (!_neutral(FuncWrapVec[i])) return _class_of(FuncWrapVec[i]);
        for (size_t i = idx + 1; i < FuncWrapVec.size(); ++i)
            if (!_neutral(FuncWrapVec[i])) return _class_of(FuncWrapVec[i]);
        return _class_of(f);
    }
    // The decomposition table is looked up with the key the scheduler used for the durations: seq rounded up to the
    // profile grid (key_seq), so a request whose length is not itself a profiled key can still be split.
    const std::vector<float>* _profile(const FuncWrap& f) {
        if (!profiling_decompse_res_dict) return nullptr;
        auto it = profiling_decompse_res_dict->find({f.name, batch_size, key_seq});
        if (it == profiling_decompse_res_dict->end() && key_seq != seq_len) it = profiling_decompse_res_dict->find({f.name, batch_size, seq_len});
        if (it == profiling_decompse_res_dict->end() || (int)it->second.size() < _factor - 1) { sub_profile_misses++; return nullptr; }
        return &it->second;
    }

  public:
    std::vector<FuncWrap> FuncWrapVec;
    const SubDict* profiling_decompse_res_dict = nullptr;  // shared, read-only (the reference copies it per sample)
    std::chrono::steady_clock::time_point sample_arrive, sample_start;
    bool started = false;
    size_t exe_num = 0;
    void *start = nullptr, *stop = nullptr, *last_launch = nullptr;
    int batch_size, seq_len;
    int key_seq = 0;            // seq_len on the profile grid (set by the scheduler; seq_len when there is no grid)
    int sub_profile_misses = 0; // GEMMs that could not be split because the decomposition table has no entry for them
    int id = 0;
    bool chunked = false;       // the launch vector is a prefill cut into chunks (entries with yield_after mark their ends)
    int n_decode_pending = 0;   // decode steps the owner still has to run for this request once the prefill vector is done
    bool merge_minor = false;  // see _neutral(); false = every entry keeps its own class (the reference's behaviour)
    void* user = nullptr;  // owner's per-request context (buffers), opaque here

    Sample(std::vector<FuncWrap>& vec, const SubDict& sub_dict, int batch_size_, int seq_len_, int factor,
           class_policy policy = CLASSIC, split_axis axis = SPLIT_OUT_COLS)
        : _factor(factor), _policy(policy), _axis(axis), FuncWrapVec(vec), profiling_decompse_res_dict(&sub_dict),
          batch_size(batch_size_), seq_len(seq_len_), key_seq(seq_len_) {
        note_status(lg_event_create(&start), "lg_event_create");
        note_status(lg_event_create(&stop), "lg_event_create");
        note_status(lg_event_create(&last_launch), "lg_event_create");
        record_arrival();
    }
    ~Sample() {
        // start/stop are handed to the recorder and destroyed by its owner
        if (last_launch) lg_event_destroy(last_launch);
    }
    Sample(const Sample&) = delete;
    Sample& operator=(const Sample&) = delete;

    bool main_empty() const { return FuncWrapVec.size() == exe_num; }
    bool empty() const { return main_empty() && _sub_empty(); }
    size_t size() const { return FuncWrapVec.size() - exe_num + _sub_size(); }
    bool sub_pending() const { return !_sub_empty(); }

    // exactly one launch left  (init.h:85-95)
    bool next_empty() const {
        if (_sub_empty()) return FuncWrapVec.size() - 1 == exe_num;
        // pieces pending: the parent is still at exe_num until its first piece has been launched
        const bool parent_consumed = _sub_exe_num > 0;
        const size_t main_left = FuncWrapVec.size() - exe_num - (parent_consumed ? 0 : 1);
        return main_left == 0 && _sub_size() == 1;
    }

    // class of the next launch and of the one after it
    int next_class() const { return _sub_empty() ? _class_at(exe_num) : _class_of(_SubFuncWrapVec[_sub_exe_num].func); }
    layer_type type() const { return _sub_empty() ? FuncWrapVec.at(exe_num).type : GEMM; }  // init.h:151-157

    // the next launch is marked as the end of a chunk (FuncWrap::yield_after); marked entries are never decomposed
    bool next_yields() const { return _sub_empty() && !main_empty() && FuncWrapVec[exe_num].yield_after; }

    // true when the next launch is the last of a run of same-class launches  (init.h:99-129)
    bool is_switch() const {
        if (next_empty()) return true;
        if (next_yields()) return true;
        if (_sub_empty()) return _class_at(exe_num) != _class_at(exe_num + 1);
        if (_sub_size() >= 2) return false;  // next two launches are pieces of the same GEMM
        const size_t after = (_sub_exe_num > 0) ? exe_num : exe_num + 1;
        return _class_of(_SubFuncWrapVec[_sub_exe_num].func) != _class_at(after);
    }

    // Stand-alone milliseconds of the launches at the head of this request that may run next to a primary segment of class
    // `cls`: everything up to the next entry of that class (at most `limit` entries are looked at).
    float run_ahead_duration(int cls, int limit = 256) const {
        float t = 0.f;
        for (size_t i = _sub_exe_num; i < _SubFuncWrapVec.size(); ++i) {
            if (_class_of(_SubFuncWrapVec[i].func) == cls) return t;
            t += _SubFuncWrapVec[i].func.duration;
        }
        const size_t first = exe_num + ((!_sub_empty() && _sub_exe_num == 0) ? 1 : 0);  // pending pieces stand for their parent
        for (size_t i = first; i < FuncWrapVec.size() && (int)(i - first) < limit; ++i) {
            if (_class_at(i) == cls) break;
            t += FuncWrapVec[i].duration;
        }
        return t;
    }

    // may not co-run with a primary segment of class `cls`  (init.h:131-149)
    bool is_same_class(int cls) const { return next_class() == cls; }
    bool is_same_type(layer_type t) const {  // the reference's signature: classic comm / non-comm comparison
        const bool next_comm = _sub_empty() ? FuncWrapVec.at(exe_num).type == COMMUNICATION : false;
        return (t == COMMUNICATION) == next_comm;
    }

    // Launches the next entry (or piece) on DParams' stream and returns its profiled duration  (init.h:160-194).
    float dequeue(const DynamicInitParam& DParams, int is_main, float& time_planned) {
        float duration = 0.0f;
        if (empty()) return duration;
        if (!started) {
            started = true;
            record_start();
            record_gpu_start(DParams);
        }
        // a sample that changes stream must wait for its own kernels on the other stream
        // (the event is recorded on the old stream only now, at the switch: it then also covers whatever other requests
        // have launched there since, which only orders more, and the common case of no switch costs no event at all)
        if (_last_stream >= 0 && _last_stream != DParams.stream_id) {
            note_status(lg_event_record(last_launch, _last_stream_handle), "lg_event_record");
            note_status(lg_stream_wait_event(DParams.stream, last_launch), "lg_stream_wait_event");
        }
        const bool last = next_empty();
        if (!_sub_empty()) {
            if (_sub_exe_num == 0) exe_num++;  // the first piece consumes the parent GEMM
            Piece& p = _SubFuncWrapVec.at(_sub_exe_num);
            p.func.callback(DParams);
            duration = p.func.duration;
            _sub_exe_num++;
            if (_sub_empty()) _sub_clear();
        } else {
            FuncWrap& f = FuncWrapVec.at(exe_num);
            f.callback(DParams);
            duration = f.duration;
            if (is_main == 0 && f.type == COMMUNICATION) duration = time_planned;  // init.h:185-188
            exe_num++;
        }
        _last_stream = DParams.stream_id;
        _last_stream_handle = DParams.stream;
        if (last) record_gpu_stop(DParams);
        return duration;
    }

    recorder get_recording() const { return recorder{time_cpu_elapsed(), start, stop, batch_size, seq_len, sample_arrive}; }

    // profiled duration of the next launch  (init.h:200-215)
    float duration(int is_main, float& time_planned) const {
        if (_sub_empty()) {
            const FuncWrap& f = FuncWrapVec.at(exe_num);
            if (is_main == 0 && f.type == COMMUNICATION) return time_planned;
            return f.duration;
        }
        return _SubFuncWrapVec.at(_sub_exe_num).func.duration;
    }

    // Tries to split the next GEMM (or its pending remainder) so that the first piece fits into time_planned
    // (init.h:226-259).  On success the sub-queue holds [piece that fits, remainder].
    bool possible_duration(float& time_planned) {
        if (_factor < 2) return false;
        if (_sub_empty()) {
            const FuncWrap& parent = FuncWrapVec.at(exe_num);
            if (!parent.args_gemm.valid) return false;
            const std::vector<float>* vec = _profile(parent);
            if (!vec) return false;
            for (int i = _factor - 2; i >= 0; i--) {
                if (time_planned >= (*vec)[i]) {
                    const int n_run = i + 1, remain = _factor - n_run;
                    _sub_clear();
                    _SubFuncWrapVec.push_back({decompose_callback(parent, _factor, n_run, (*vec)[i], 0, _axis), 0, n_run});
                    _SubFuncWrapVec.push_back({decompose_callback(parent, _factor, remain, (*vec)[remain - 1], n_run, _axis), n_run, remain});
                    return true;
                }
            }
            return false;
        }
        // a remainder is pending: split it again
        const Piece cur = _SubFuncWrapVec.at(_sub_exe_num);
        if (_sub_size() != 1 || cur.count < 2) return false;
        // the parent's descriptor: pieces are always cut from the full GEMM, so offsets stay exact
        const FuncWrap& parent = FuncWrapVec.at(exe_num - 1);
        const std::vector<float>* vec = _profile(parent);
        if (!vec) return false;
        for (int i = cur.count - 2; i >= 0; i--) {
            if (time_planned >= (*vec)[i]) {
                const int n_run = i + 1, remain = cur.count - n_run;
                const size_t keep = _sub_exe_num;
                _SubFuncWrapVec.resize(keep);
                _SubFuncWrapVec.push_back({decompose_callback(parent, _factor, n_run, (*vec)[i], cur.start, _axis), cur.start, n_run});
                _SubFuncWrapVec.push_back({decompose_callback(parent, _factor, remain, (*vec)[remain - 1], cur.start + n_run, _axis),
                                           cur.start + n_run, remain});
                return true;
            }
        }
        return false;
    }

    void record_arrival() { sample_arrive = std::chrono::steady_clock::now(); }
    void record_start() { sample_start = std::chrono::steady_clock::now(); }
    void record_gpu_start(const DynamicInitParam& D) { note_status(lg_event_record(start, D.stream), "lg_event_record"); }
    void record_gpu_stop(const DynamicInitParam& D) { note_status(lg_event_record(stop, D.stream), "lg_event_record"); }
    double time_cpu_elapsed() const { return std::chrono::duration<double>(sample_start - sample_arrive).count(); }
};

}  // namespace liger
