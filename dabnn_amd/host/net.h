// bnn::Net (dabnn/net.h:22-68): loads a .dab model, owns the blobs, runs the
// layers in order.  Public surface as in the reference -- create / read /
// read_buf / run / get_blob and the flags optimize / run_fconv / strict --
// plus a batch size, which the reference does not have (dabnn/net.cpp:64-65).
//
// All blobs live in device memory; run() takes a HOST pointer to
// batch x H x W x C floats (NHWC) like the reference's run(void*), uploads it,
// enqueues every layer on the net's stream and waits.  run_device() takes a
// device pointer and reads the input in place (as the reference's run wraps
// its host pointer without a copy).
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "layer.h"
#include "mat.h"

namespace bnn {

class BNN_API Net : public std::enable_shared_from_this<Net> {
   public:
    static std::shared_ptr<Net> create();
    ~Net();

    void set_batch(int batch);  // before read(); default 1
    int batch() const { return batch_; }
    const std::string &input_name() const { return input_name_; }
    void read(const std::string &path);
    void read_buf(const void *ptr);
    void read_buf(const void *ptr, size_t len);  // the same, with every offset of the model checked against len
    void run(const void *host_input);
    // The layers read device_input where it lies, which must stay valid and unchanged until the call returns (256-byte
    // aligned, as hipMalloc gives it; anything else is copied into the net's own input blob).  The HIP graph holds
    // the address it was captured with: the same buffer run after run replays it, another buffer makes the net
    // capture again, and from the third such change on the net copies every input into its own blob instead.
    // nullptr: the input blob already holds the input.
    void run_device(const void *device_input);
    // The blob with its host mirror up to date (dabnn/net.cpp:288-290): `data`, operator[] ... read what the last
    // run left on the device.
    std::shared_ptr<Mat> get_blob(const std::string &name);
    // The same blob without the device-to-host copy (what the layers and the C ABI use).
    std::shared_ptr<Mat> blob(const std::string &name);
    bool has_blob(const std::string &name) const { return mat_map_.count(name) != 0; }
    std::vector<std::string> layer_descriptions() const;

    // optimize: true picks the direct 3x3 kernel where it applies, false sends every
    // BinConv through im2col + bgemm (the reference's switch between its optimised and
    // plain kernels; both settings give identical outputs).
    bool optimize = true;
    bool run_fconv = true;
    bool strict = true;

    // Replay the layer sequence as one HIP graph from the third run on (the first two run eagerly so that every
    // kernel has been launched once outside capture).  Launch overhead dominates at batch 1; switch off to
    // debug or when layers are added between runs.
    bool use_graph = true;

    // per-layer-type milliseconds of the last runs when profiling (BNN_BENCHMARK of the reference)
    bool profile = false;
    std::map<std::string, double> layer_time_;
    std::string time_report() const;

    void *stream() const { return stream_; }
    void add_mat(const std::string &name, std::shared_ptr<Mat> mat);
    std::map<std::string, std::shared_ptr<Mat>> mat_map_;
    // blobs of the model that the optimized layer list never writes (name -> why); get_blob names the reason
    std::map<std::string, std::string> elided_;

   private:
    Net();
    void prepare(const void *model_buf, size_t len);
    void fuse_binconv_epilogues();
    std::weak_ptr<Net> get_weak() { return shared_from_this(); }
    std::vector<std::shared_ptr<Layer>> layers;
    std::map<std::string, std::vector<uint32_t>> shapes_;  // NHWC with N = 1, as stored in the model
    std::string input_name_;
    std::vector<uint8_t> file_;  // owns the model bytes when read from a path
    int batch_ = 1;
    void *stream_ = nullptr;
    bool prepared_ = false;
    int runs_ = 0;
    void *graph_exec_ = nullptr;
    void *input_own_dev_ = nullptr;       // the input blob's own allocation
    const void *graph_input_ = nullptr;   // the input address the graph's kernels hold
    int input_rebinds_ = 0;               // captures thrown away because the caller's buffer changed
    bool copy_input_ = false;             // the caller's buffers keep changing: copy into the own blob
    void bind_input(const void *device_input);
    bool layers_write_input();
    void launch_layers();
};

}  // namespace bnn
