// liger_main.cpp -- command-line driver: profile, then serve a request trace with and without interleaving.
//
// Counterpart of the reference's main.cu (:10-55) and src/test_schedule.h (test_profile :81-104, test_schedule :20-48,
// test_no_schedule :51-78) without the MPI / NCCL bootstrap: one process, one GPU, one tensor-parallel shard.
// Arguments (all optional, in the reference's order, main.cu:24-31):
//   max_batch max_seq head_num size_per_head layer_num factor arrival_rate [world_size] [requests]
#include <cstdio>
#include <cstdlib>
#include <string>

#include "scheduler.h"

using namespace liger;

int main(int argc, char** argv) {
    int max_batch_size = 2, max_seq_len = 128, head_num = 96, size_per_head = 128, layer_num = 4, factor = 8;
    int arr_rate = 80, world_size = 2, requests = 150;
    int* slots[] = {&max_batch_size, &max_seq_len, &head_num, &size_per_head, &layer_num, &factor, &arr_rate, &world_size, &requests};
    for (int i = 1; i < argc && i <= 9; ++i) *slots[i - 1] = atoi(argv[i]);
    const int rq_interval = (int)(1e6 / arr_rate);  // microseconds, main.cu:33

    StaticInitParam SParams(0, world_size, LG_F16);
    BertInitParam P(max_batch_size, max_seq_len, head_num, size_per_head, layer_num, 0, factor, rq_interval);
    P.fused = 1;
    P.weight_layout = 1;
    const int hidden = head_num * size_per_head;
    half* workspace = dev_alloc<half>(Bert_Encoder<half>::workspace_elems(P, SParams, max_batch_size, max_seq_len));
    Bert_Model<half> model(P, SParams, hidden, hidden, workspace);
    model.init_weights(0);
    P.kernel_num = model.kernels_per_layer();
    half* input = dev_alloc<half>((size_t)max_batch_size * max_seq_len * hidden);
    half* output = dev_alloc<half>((size_t)max_batch_size * max_seq_len * hidden);
    dev_fill_normal(input, (int64_t)max_batch_size * max_seq_len * hidden, 0, 7, 0.f, 1.f);

    const std::string tag = std::to_string(world_size) + "_" + std::to_string(size_per_head) + "_" + std::to_string(head_num) + "_" +
                            std::to_string(max_batch_size) + "_" + std::to_string(max_seq_len) + ".json";
    const std::string main_file = "./Main_" + tag, sub_file = "./Sub_" + tag;  // test_schedule.h:36-39

    {   // to collect profiling results
        Scheduler<half, Bert_Model<half>> prof(&model, P, SParams, input, output);
        prof.profile(max_batch_size, max_batch_size + 1, 16, max_seq_len + 1, main_file, sub_file, 4);
        printf("profiled %zu kernels, %zu decomposable\n", prof.profiling_res_dict.size(), prof.profiling_decompse_res_dict.size());
    }
    for (int liger_on = 1; liger_on >= 0; --liger_on) {   // running with Liger, then without
        Scheduler<half, Bert_Model<half>> sched(&model, P, SParams, input, output, main_file, sub_file);
        sched.policy = RESOURCE;
        sched.seq_bucket = 4;
        sched.make_pool(8, max_batch_size);
        sched.serving(sched.reference_trace(requests));
        if (liger_on) sched.run_stream_sync(); else sched.run_sequential();
        printf("---- %s ----\n", liger_on ? "run_stream_sync" : "run_sequential");
        sched.output_recording();
    }
    if (first_error()) {
        fprintf(stderr, "error: %s\n", error_text().c_str());
        return 1;
    }
    return 0;
}
