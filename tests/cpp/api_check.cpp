// A C++ user of the host layer, written against the reference's names: load an `.espdl` file with
// fbs::FbsLoader, build a dl::Model, run its embedded test vectors, then run it again by hand and read the
// output back.  Exit code 0 = everything matched.  Built and run by tests/test_gpu_cpp_api.py.
#include <cstdio>
#include <cstring>
#include <vector>

#include "dl_model_base.hpp"
#include "fbs_loader.hpp"

int main(int argc, char **argv)
{
    if (argc < 3) {
        std::fprintf(stderr, "usage: %s model.espdl round_mode(0|1)\n", argv[0]);
        return 2;
    }
    fbs::FbsLoader loader(argv[1], fbs::MODEL_LOCATION_IN_SDCARD);
    fbs::FbsModel *graph = loader.load();
    if (!graph) {
        std::fprintf(stderr, "load failed: %s\n", loader.last_error().c_str());
        return 3;
    }
    const dl::round_mode_t rm = argv[2][0] == '1' ? dl::ROUND_MODE_HALF_EVEN : dl::ROUND_MODE_HALF_UP;
    dl::Model model(graph, /*batch=*/1, rm);
    if (model.test() != ESP_OK)
        return 4;

    // the same by hand: test input -> run -> compare with the test output
    int rc = 0;
    for (const std::string &in_name : graph->get_graph_inputs()) {
        dl::TensorBase *t = graph->get_test_input_tensor(in_name);
        if (!t || !model.get_input(in_name)->copy_from_host(t->data, t->get_bytes()))
            rc = 5;
        delete t;
    }
    model.run();
    for (const std::string &out_name : graph->get_test_outputs_name()) {
        dl::TensorBase *want = graph->get_test_output_tensor(out_name);
        dl::TensorBase *got = model.get_intermediate(out_name);
        std::vector<char> host(want->get_bytes());
        if (!got || got->get_bytes() != want->get_bytes() || !got->copy_to_host(host.data(), host.size()) ||
            std::memcmp(host.data(), want->data, host.size()) != 0) {
            std::fprintf(stderr, "output %s differs\n", out_name.c_str());
            rc = 6;
        }
        delete want;
    }
    std::printf("%s: %s\n", argv[1], rc == 0 ? "ok" : "FAILED");
    delete graph;
    return rc;
}
