// The loader-free part of the host layer, used the way the reference's API tests use it
// (test_apps/esp-dl/main/test_dl_api.cpp:20-335): Module::run on bare tensors (one input / one output,
// several inputs), StreamingCache::reset, Model::run(stage_num, stage_index), Model::reset, and what a
// failed forward reports.  `shapes` runs the checks that need no device (get_output_shape rules);
// `device <model.espdl>` runs the rest.  Exit code 0 = everything matched; the first failing check is
// printed.  Built by esp-dl_amd/build.py, run by tests/test_module_api.py.
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "dl_model_base.hpp"
#include "dl_module_creator.hpp"
#include "fbs_loader.hpp"

using namespace dl;

static int g_failed = 0;
#define CHECK(cond)                                                           \
    do {                                                                      \
        if (!(cond)) {                                                        \
            std::fprintf(stderr, "%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); \
            g_failed++;                                                       \
        }                                                                     \
    } while (0)

typedef std::vector<int> shape_t;

static shape_t out_shape(module::Module &m, shape_t in)
{
    std::vector<shape_t> ins = {in};
    std::vector<shape_t> outs = m.get_output_shape(ins);
    return outs.empty() ? shape_t() : outs[0];
}

// Reshape / Squeeze shape rules (esp-dl/dl/module/include/dl_module_reshape.hpp:36-75,
// dl_module_squeeze.hpp:33-70), and how the batch dimension enters them.
static void check_shapes()
{
    using module::ShapeView;
    {
        ShapeView r("r", ShapeView::RESHAPE, {1, -1, 8});
        CHECK(out_shape(r, {1, 4, 4, 8}) == shape_t({1, 16, 8}));
        CHECK(out_shape(r, {5, 4, 4, 8}) == shape_t({5, 16, 8})); // leading 1 of the exported target = the batch
    }
    {
        ShapeView r("r", ShapeView::RESHAPE, {-1, 8}); // folds the leading dimension: the target as written
        CHECK(out_shape(r, {1, 4, 4, 8}) == shape_t({16, 8}));
        CHECK(out_shape(r, {3, 4, 4, 8}) == shape_t({48, 8}));
        CHECK(out_shape(r, {1, 3, 3, 3}).empty()); // 27 elements are not a multiple of 8
    }
    {
        ShapeView r("r", ShapeView::RESHAPE, {16, 8});
        CHECK(out_shape(r, {1, 4, 4, 8}) == shape_t({16, 8}));
        CHECK(out_shape(r, {2, 4, 4, 8}).empty()); // 256 elements into a 128-element target: no shape
    }
    {
        ShapeView r("r", ShapeView::RESHAPE, {0, 0, -1}); // 0 copies the input extent
        CHECK(out_shape(r, {7, 4, 4, 8}) == shape_t({7, 4, 32}));
    }
    {
        ShapeView r("r", ShapeView::RESHAPE, {1, 5, 5});
        CHECK(out_shape(r, {1, 4, 4, 2}).empty());
        ShapeView two("r", ShapeView::RESHAPE, {-1, -1, 4});
        CHECK(out_shape(two, {1, 4, 4, 2}).empty());
    }
    {
        ShapeView s("s", ShapeView::SQUEEZE, {});
        CHECK(out_shape(s, {1, 1, 40, 120}) == shape_t({40, 120})); // batch of one: every 1 goes
        CHECK(out_shape(s, {6, 1, 40, 120}) == shape_t({6, 40, 120}));
        ShapeView a("s", ShapeView::SQUEEZE, {1});
        CHECK(out_shape(a, {1, 1, 40, 120}) == shape_t({1, 40, 120}));
        CHECK(out_shape(a, {1, 2, 40, 120}) == shape_t({1, 2, 40, 120})); // an axis whose extent is not 1 stays
        ShapeView u("u", ShapeView::UNSQUEEZE, {1, -1});
        CHECK(out_shape(u, {3, 40}) == shape_t({3, 1, 40, 1}));
    }
    {
        // errors are counted: a caller that cannot see stderr can still tell that something was logged
        const long before = error_log_count().load();
        DL_LOGE("check", "this line is expected (%d)", 1);
        CHECK(error_log_count().load() == before + 1);
    }
}

static std::vector<int8_t> random_bytes(size_t n, unsigned seed)
{
    std::mt19937 rng(seed);
    std::vector<int8_t> v(n);
    for (auto &x : v)
        x = (int8_t)((int)(rng() & 255) - 128);
    return v;
}

static std::vector<int8_t> download(TensorBase *t)
{
    std::vector<int8_t> host(t->get_bytes());
    CHECK(t->copy_to_host(host.data(), host.size()));
    return host;
}

// "Test dl module API: run()": Relu with one input and one output, Add with two inputs (the second
// broadcast over the leading dimensions), on bare device tensors without a model.
static void check_module_run()
{
    const shape_t shape = {1, 3, 64, 64};
    std::vector<int8_t> a = random_bytes(3 * 64 * 64, 1), b = random_bytes(64, 2);
    // keep the sums inside int8 so that the reference's own check (in1 + in2 == out) is meaningful
    for (auto &x : a)
        x = (int8_t)(x / 2);
    for (auto &x : b)
        x = (int8_t)(x / 2);
    TensorBase input1(shape, a.data(), 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
    TensorBase input2({1, 1, 1, 64}, b.data(), 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
    TensorBase output(shape, nullptr, 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);

    module::Relu relu_op("relu", MODULE_NON_INPLACE, QUANT_TYPE_SYMM_8BIT);
    relu_op.run(&input1, &output);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    std::vector<int8_t> got = download(&output);
    bool ok = true;
    for (size_t i = 0; i < got.size(); i++)
        ok = ok && got[i] == (a[i] > 0 ? a[i] : 0);
    CHECK(ok);

    module::Add add_op("add", MODULE_NON_INPLACE, QUANT_TYPE_SYMM_8BIT);
    add_op.run({&input1, &input2}, {&output});
    CHECK(hipDeviceSynchronize() == hipSuccess);
    got = download(&output);
    ok = true;
    for (size_t i = 0; i < got.size(); i++)
        ok = ok && got[i] == (int8_t)(a[i] + b[i % 64]);
    CHECK(ok);

    // a host tensor handed to a device module is an error that is logged and counted, not a crash
    TensorBase host_in(shape, a.data(), 0, DATA_TYPE_INT8);
    const long before = error_log_count().load();
    relu_op.run(&host_in, &output);
    CHECK(error_log_count().load() > before);
}

// "Test dl module API: StreamingCache reset()"
static void check_streaming_cache_reset()
{
    TensorBase input({1, 2, 4, 4}, nullptr, 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
    TensorBase output({1, 3, 4, 4}, nullptr, 0, DATA_TYPE_INT8, true, MALLOC_CAP_DEVICE);
    module::StreamingCache cache_op("streaming_cache", 2, 1, QUANT_TYPE_NONE);
    input.memset(5);
    cache_op.run(&input, &output);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    std::vector<int8_t> first = download(&output);
    input.memset(10);
    cache_op.run(&input, &output);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    std::vector<int8_t> second = download(&output);
    CHECK(first != second); // the cache was updated
    cache_op.reset();
    input.memset(5);
    cache_op.run(&input, &output);
    CHECK(hipDeviceSynchronize() == hipSuccess);
    std::vector<int8_t> third = download(&output);
    CHECK(first == third);
    for (int i = 0; i < 16; i++)
        CHECK(third[i] == 0); // the first frame comes from the cleared cache
}

// "Test dl model API: run()" (stage by stage) and "reset()"
static void check_model_stages(const char *path)
{
    fbs::FbsLoader loader(path, fbs::MODEL_LOCATION_IN_SDCARD);
    fbs::FbsModel *graph = loader.load();
    CHECK(graph != nullptr);
    if (!graph)
        return;
    Model model(graph, /*batch=*/2);
    CHECK(model.get_module_count() >= 3);
    std::vector<std::vector<int8_t>> saved;
    unsigned seed = 11;
    for (auto &kv : model.get_inputs()) {
        saved.push_back(random_bytes(kv.second->get_bytes(), seed++));
        CHECK(kv.second->copy_from_host(saved.back().data(), saved.back().size()));
    }
    model.run();
    CHECK(!model.last_run_failed());
    std::vector<std::vector<int8_t>> whole;
    for (auto &kv : model.get_outputs())
        whole.push_back(download(kv.second));

    model.reset(); // clears every activation; the inputs have to be written again
    size_t k = 0;
    for (auto &kv : model.get_inputs())
    {
            CHECK(kv.second->copy_from_host(saved[k].data(), saved[k].size()));
            k++;
        }
    for (auto &kv : model.get_outputs()) {
        std::vector<int8_t> cleared = download(kv.second);
        bool all_zero = true;
        for (int8_t v : cleared)
            all_zero = all_zero && v == 0;
        CHECK(all_zero);
    }
    model.run(3, 0);
    model.run(3, 1);
    model.run(3, 2);
    CHECK(!model.last_run_failed());
    k = 0;
    for (auto &kv : model.get_outputs())
    {
            CHECK(download(kv.second) == whole[k]);
            k++;
        }
    // an out-of-range stage is refused and reported
    const long before = error_log_count().load();
    model.run(3, 3);
    CHECK(error_log_count().load() > before);

    // third run after reset with the same inputs equals the first
    model.reset();
    k = 0;
    for (auto &kv : model.get_inputs())
    {
            CHECK(kv.second->copy_from_host(saved[k].data(), saved[k].size()));
            k++;
        }
    model.run();
    k = 0;
    for (auto &kv : model.get_outputs())
    {
            CHECK(download(kv.second) == whole[k]);
            k++;
        }
    delete graph;
}

int main(int argc, char **argv)
{
    if (argc >= 2 && std::strcmp(argv[1], "shapes") == 0) {
        check_shapes();
    } else if (argc >= 3 && std::strcmp(argv[1], "device") == 0) {
        check_module_run();
        check_streaming_cache_reset();
        check_model_stages(argv[2]);
    } else {
        std::fprintf(stderr, "usage: %s shapes | device model.espdl\n", argv[0]);
        return 2;
    }
    std::printf("%s: %s\n", argv[1], g_failed == 0 ? "ok" : "FAILED");
    return g_failed == 0 ? 0 : 1;
}
