// extern "C" face of bnn::Net; exceptions become error codes.
#include "../../include/dabnn_net.h"

#include <cstring>
#include <stdexcept>
#include <string>
#include <vector>

#include "model.h"
#include "net.h"

struct dabnet {
    std::shared_ptr<bnn::Net> net;
    std::vector<std::string> descs;
    std::string report;
};

static thread_local std::string g_error;

template <class F>
static int guarded(F &&f) {
    try {
        f();
        return DABNET_OK;
    } catch (const std::invalid_argument &e) {
        g_error = e.what();
        return DABNET_EINVALID;
    } catch (const std::out_of_range &e) {
        g_error = e.what();
        return DABNET_EKEY;
    } catch (const std::exception &e) {
        g_error = e.what();
        return DABNET_ERUNTIME;
    } catch (...) {
        g_error = "unknown exception";
        return DABNET_ERUNTIME;
    }
}

extern "C" {

const char *dabnet_last_error(void) { return g_error.c_str(); }

dabnet_t *dabnet_create(void) {
    dabnet_t *h = nullptr;
    const int rc = guarded([&] {
        h = new dabnet;
        h->net = bnn::Net::create();
    });
    if (rc != DABNET_OK) {
        delete h;
        return nullptr;
    }
    return h;
}

void dabnet_destroy(dabnet_t *net) { delete net; }

int dabnet_set_batch(dabnet_t *net, int batch) {
    return guarded([&] { net->net->set_batch(batch); });
}

int dabnet_set_flags(dabnet_t *net, int optimize, int run_fconv, int strict) {
    return guarded([&] {
        net->net->optimize = optimize != 0;
        net->net->run_fconv = run_fconv != 0;
        net->net->strict = strict != 0;
    });
}

int dabnet_set_use_graph(dabnet_t *net, int on) {
    return guarded([&] { net->net->use_graph = on != 0; });
}

int dabnet_set_profile(dabnet_t *net, int on) {
    return guarded([&] {
        net->net->profile = on != 0;
        net->net->layer_time_.clear();
    });
}

const char *dabnet_time_report(dabnet_t *net) {
    net->report = net->net->time_report();
    return net->report.c_str();
}

int dabnet_read_file(dabnet_t *net, const char *path) {
    return guarded([&] {
        if (!path) throw std::invalid_argument("null path");
        net->net->read(path);
    });
}

int dabnet_read_buf(dabnet_t *net, const void *buf, size_t len) {
    return guarded([&] {
        if (!buf || len < 8) throw std::invalid_argument("model buffer too small");
        net->net->read_buf(buf, len);
    });
}

int dabnet_check_model(const void *buf, size_t len, int run_fconv) {
    return guarded([&] {
        if (!buf || len < 8) throw std::invalid_argument("model buffer too small");
        bnn::ModelDesc model = bnn::parse_model(buf, len);
        bnn::check_model(model, run_fconv != 0);
    });
}

int dabnet_run(dabnet_t *net, const float *host_input) {
    return guarded([&] { net->net->run(host_input); });
}

int dabnet_run_device(dabnet_t *net, const float *device_input) {
    return guarded([&] {
        if (!device_input) throw std::runtime_error("run_device: null input");
        net->net->run_device(device_input);
    });
}

const char *dabnet_input_name(dabnet_t *net) { return net->net->input_name().c_str(); }

int dabnet_blob_info(dabnet_t *net, const char *name, int shape[4], int *is_bit, size_t *bytes) {
    return guarded([&] {
        auto m = net->net->blob(name ? name : "");
        if (shape) shape[0] = m->n, shape[1] = m->h, shape[2] = m->w, shape[3] = m->c;
        if (is_bit) *is_bit = m->data_type == bnn::DataType::Bit;
        if (bytes) *bytes = m->bytes();
    });
}

int dabnet_get_blob(dabnet_t *net, const char *name, void *host_out, size_t bytes) {
    return guarded([&] {
        auto m = net->net->blob(name ? name : "");
        if (!host_out) throw std::runtime_error("get_blob: null destination");
        m->download(host_out, bytes);
    });
}

int dabnet_num_layers(dabnet_t *net) {
    net->descs = net->net->layer_descriptions();
    return (int)net->descs.size();
}

const char *dabnet_layer_desc(dabnet_t *net, int index) {
    if (net->descs.empty()) net->descs = net->net->layer_descriptions();
    if (index < 0 || index >= (int)net->descs.size()) return "";
    return net->descs[index].c_str();
}

}  // extern "C"
