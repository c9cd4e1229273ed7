// The reference's own way of using a network, compiled against this library's C++ headers: the body of
// tests/net_test.cpp:29-50 (optimize = false against optimize = true through Mat::operator==) and the accessors its
// other callers use ((*blob)[i] in tests/net_test.cpp:63-65, static_cast<float *>(*blob) and total() in
// dabnn/jni/JavaWrapper.cpp:56-60, blob->data and data_type in binaries/run.cpp:41-50), on a model file given on the
// command line.  Prints the first values of the blob for the caller to compare; exit status 0 when every check holds.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../dabnn_amd/host/net.h"

#define CHECK(cond)                                                          \
    do {                                                                     \
        if (!(cond)) {                                                       \
            std::fprintf(stderr, "%s:%d: CHECK(%s) failed\n", __FILE__, __LINE__, #cond); \
            return 1;                                                        \
        }                                                                    \
    } while (0)

int main(int argc, char **argv) {
    if (argc < 4) {
        std::fprintf(stderr, "usage: %s model.dab blob_name input_floats\n", argv[0]);
        return 2;
    }
    const std::string path = argv[1], blob_name = argv[2];
    const size_t n_in = (size_t)std::atol(argv[3]);
    std::vector<float> input(n_in, 1.0f);  // FORZ(i, 3 * 224 * 224) { input[i] = 1; }

    std::shared_ptr<bnn::Mat> blob1, blob2;
    {
        auto net = bnn::Net::create();
        net->optimize = false;
        net->read(path);
        net->run(input.data());
        blob1 = net->get_blob(blob_name);
    }
    {
        auto net = bnn::Net::create();
        net->optimize = true;
        net->read(path);
        net->run(input.data());
        blob2 = net->get_blob(blob_name);
    }
    // the blobs outlive their nets, as in the reference's test
    CHECK(*blob1 == *blob2);  // ASSERT_EQ(*blob1, *blob2)
    CHECK(blob1->data_type == bnn::DataType::Float);
    CHECK(blob2->total() > 3);

    auto net = bnn::Net::create();
    net->read(path);
    net->run(input.data());
    const auto blob = net->get_blob(blob_name);
    const float *as_ptr = static_cast<float *>(*blob);       // JavaWrapper.cpp:59-60
    const float *raw = static_cast<float *>(blob->data);     // binaries/run.cpp:41
    CHECK(as_ptr == raw);
    for (int i = 0; i < 3; ++i) {
        CHECK((*blob)[i] == as_ptr[i]);                       // tests/net_test.cpp:63-65
        CHECK(std::abs((*blob)[i] - (*blob2)[i]) <= 1e-5f);
    }
    CHECK(blob->point<float>(0, 0) == as_ptr);
    std::printf("total %zu\n", blob->total());
    for (size_t i = 0; i < blob->total() && i < 8; ++i) std::printf("v %zu %.9g\n", i, (*blob)[(int)i]);
    std::ostringstream os;
    os << *blob;
    CHECK(os.str().find("channels") != std::string::npos);

    // a Bit blob (the packed input of a binary convolution, named as in dabnn/layers/BinConv.cpp:24) compares word
    // by word
    if (argc > 4) {
        const auto bits = net->get_blob(argv[4]);
        CHECK(bits->data_type == bnn::DataType::Bit && bits->elemsize == 8 && bits->elem_c == bits->c * 64);
        auto other = bnn::Net::create();
        other->read(path);
        other->run(input.data());
        CHECK(*bits == *other->get_blob(argv[4]));
        const uint64_t *words = static_cast<uint64_t *>(*bits);
        std::printf("w0 %llu\n", (unsigned long long)words[0]);
    }
    // a second run with another input: the Mat in hand shows the new values after get_blob
    for (auto &v : input) v = -0.5f;
    net->run(input.data());
    const auto again = net->get_blob(blob_name);
    CHECK(again.get() == blob.get());
    CHECK(!(*again == *blob2) || blob->total() == 0);
    bool threw = false;
    try {
        bnn::Net::create()->read("/nonexistent/model.dab");
    } catch (const std::invalid_argument &) {  // dabnn/net.cpp:34-36
        threw = true;
    }
    CHECK(threw);
    threw = false;
    try {
        net->get_blob("no such blob");
    } catch (const std::out_of_range &) {
        threw = true;
    }
    CHECK(threw);
    std::printf("ok\n");
    return 0;
}
