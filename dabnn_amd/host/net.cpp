#include "net.h"

#include <algorithm>

#include <hip/hip_runtime_api.h>

#include <fstream>
#include <mutex>
#include <sstream>
#include <stdexcept>

#include "../../include/dabnn_hip_tuning.h"
#include "layers.h"
#include "model.h"

namespace bnn {

namespace {

void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

}  // namespace

// ---------------------------------------------------------------- Layer::forward with optional timing
void Layer::forward() {
    auto net = net_.lock();
    if (!net->profile) {
        forward_impl();
        return;
    }
    hipStream_t s = static_cast<hipStream_t>(net->stream());
    hipEvent_t e0, e1;
    hip_check(hipEventCreate(&e0), "hipEventCreate");
    hip_check(hipEventCreate(&e1), "hipEventCreate");
    hip_check(hipEventRecord(e0, s), "hipEventRecord");
    forward_impl();
    hip_check(hipEventRecord(e1, s), "hipEventRecord");
    hip_check(hipEventSynchronize(e1), "hipEventSynchronize");
    float ms = 0.f;
    hip_check(hipEventElapsedTime(&ms, e0, e1), "hipEventElapsedTime");
    net->layer_time_[type_] += ms;
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
}

// ---------------------------------------------------------------- Net
// Nets of one process may run on host threads of their own.  A net captures its HIP graph on its third run; device
// allocations and frees of other threads (a net being read or destroyed) and a second capture stay out of that
// window.  Kernel launches and copies of other nets do not take the lock.
static std::mutex &capture_mutex() {
    static std::mutex m;
    return m;
}

Net::Net() {
    hipStream_t s;
    hip_check(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
    stream_ = s;
}

Net::~Net() {
    std::lock_guard<std::mutex> lock(capture_mutex());
    if (graph_exec_) (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec_));
    if (input_own_dev_ && mat_map_.count(input_name_)) mat_map_[input_name_]->dev = input_own_dev_;  // freed by its Mat
    layers.clear();
    mat_map_.clear();
    if (stream_) (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
}

std::shared_ptr<Net> Net::create() {
    struct make_shared_enabler : public Net {};
    return std::make_shared<make_shared_enabler>();
}

void Net::set_batch(int batch) {
    BNN_ASSERT(!prepared_, "set_batch must be called before the model is read");
    BNN_ASSERT(batch > 0, "batch must be positive");
    batch_ = batch;
}

void Net::read(const std::string &path) {
    // dabnn/net.cpp:32-44 maps the file; here the bytes are copied once and the
    // tensors uploaded to the device, so the file buffer can go afterwards.
    std::ifstream f(path, std::ios::binary | std::ios::ate);
    if (!f) throw std::invalid_argument("Open file error " + path);
    const std::streamsize size = f.tellg();
    if (size < 8) throw std::invalid_argument("Not a dabnn model: " + path);
    f.seekg(0);
    file_.resize((size_t)size);
    if (!f.read(reinterpret_cast<char *>(file_.data()), size)) throw std::invalid_argument("Read file error " + path);
    prepare(file_.data(), file_.size());
    file_.clear();
    file_.shrink_to_fit();
}

void Net::read_buf(const void *ptr) {
    // the reference's signature (dabnn/net.cpp:46): the extent of the buffer is unknown, so offsets are only kept
    // from wrapping around; callers that know the size use read_buf(ptr, len)
    BNN_ASSERT(ptr != nullptr, "read_buf: null model buffer");
    prepare(ptr, SIZE_MAX);
}

void Net::read_buf(const void *ptr, size_t len) {
    BNN_ASSERT(ptr != nullptr, "read_buf: null model buffer");
    prepare(ptr, len);
}

void Net::add_mat(const std::string &name, std::shared_ptr<Mat> mat) { mat_map_[name] = mat; }

std::shared_ptr<Mat> Net::get_blob(const std::string &name) {
    auto m = blob(name);
    m->sync_to_host();
    return m;
}

std::shared_ptr<Mat> Net::blob(const std::string &name) {
    auto it = mat_map_.find(name);
    if (it == mat_map_.end()) {
        auto gone = elided_.find(name);
        if (gone != elided_.end())
            throw std::runtime_error("blob " + name + " is not produced: " + gone->second + "; read the model with optimize = false to get it");
        throw std::out_of_range("Key " + name + " not found.");  // StrKeyMap::at, common/StrKeyMap.h
    }
    return it->second;
}

void Net::prepare(const void *buf, size_t len) {
    std::lock_guard<std::mutex> lock(capture_mutex());
    BNN_ASSERT(!prepared_, "a Net can be read once");
    BNN_ASSERT(!(strict && !run_fconv), "fconv must be run in strict mode");
    // parse (bounds-checked) and check the whole model on the host before anything is allocated on the device
    ModelDesc model = parse_model(buf, len);
    check_model(model, run_fconv);
    for (const auto &kv : model.shapes) shapes_[kv.first] = kv.second;
    // every blob of the batch must stay within the int extents of Mat and of the kernels' pixel counts
    for (const auto &kv : model.shapes) {
        if (kv.second.size() != 4) continue;
        const uint64_t per_image = (uint64_t)kv.second[1] * kv.second[2] * kv.second[3];
        BNN_ASSERT(per_image * (uint64_t)batch_ < (1ull << 31), "blob " + kv.first + " is too large at batch " + std::to_string(batch_));
    }

    // inputs: the first one only (dabnn/net.cpp:59-70)
    {
        const InputDesc &in = model.inputs[0];
        input_name_ = in.name;
        add_mat(input_name_, std::make_shared<Mat>(batch_, in.shape[1], in.shape[2], in.shape[3], DataType::Float, input_name_));
        input_own_dev_ = mat_map_[input_name_]->dev;
    }

    // initializers (dabnn/net.cpp:72-138), uploaded to the device
    for (const TensorDesc &t : model.initializers) {
        std::shared_ptr<Mat> m;
        if (t.is_bit) {
            // shape is [n][kh][kw][c]; the word count per filter may include the padding to 128 bits
            m = std::make_shared<Mat>(t.len, DataType::Bit, t.name);
            m->n = t.shape[0], m->h = t.shape[1], m->w = t.shape[2], m->c = t.shape[3] / 64, m->elem_c = t.shape[3];
            m->upload(t.data, t.len * 8);
        } else {
            if (t.shape.size() == 4)
                m = std::make_shared<Mat>((int)t.shape[0], (int)t.shape[1], (int)t.shape[2], (int)t.shape[3], DataType::Float, t.name);
            else
                m = std::make_shared<Mat>((size_t)t.shape[0], DataType::Float, t.name);
            m->upload(t.data, t.len * 4);
        }
        add_mat(t.name, m);
    }

    auto new_output = [&](const std::string &name, DataType type = DataType::Float, int images = 0) {
        const auto &s = model.shapes.at(name);
        if (!has_blob(name))
            add_mat(name, std::make_shared<Mat>(images ? images : batch_, (int)s[1], (int)s[2], (int)s[3], type, name));
    };
    auto alias_output = [&](const std::string &output, const std::string &input) {  // ADD_INPLACE_LAYER
        add_mat(output, blob(input));
    };

    for (const LayerDesc &l : model.layers) {
        switch (l.type) {
            case kFpConv2D:
            case kBinConv2D: {
                new_output(l.outputs[0]);
                if (l.type == kBinConv2D) {
                    layers.push_back(std::make_shared<BinConv>(get_weak(), l.name, l.inputs[0], l.weight, l.outputs[0], l.pad_h,
                                                               l.pad_w, l.stride_h, l.stride_w));
                } else if (run_fconv) {
                    if (!l.bias.empty())
                        layers.push_back(std::make_shared<FloatConv>(get_weak(), l.name, l.inputs[0], l.weight, l.bias, l.outputs[0],
                                                                     l.pad_h, l.pad_w, l.stride_h, l.stride_w, l.dil_h));
                    else
                        layers.push_back(std::make_shared<FloatConv>(get_weak(), l.name, l.inputs[0], l.weight, l.outputs[0], l.pad_h,
                                                                     l.pad_w, l.stride_h, l.stride_w, l.dil_h));
                }
                break;
            }
            case kAffine:
                alias_output(l.outputs[0], l.inputs[0]);
                layers.push_back(std::make_shared<Affine>(get_weak(), l.name, l.inputs[0], l.a, l.b));
                break;
            case kAdd:
                alias_output(l.outputs[0], l.inputs[0]);
                layers.push_back(std::make_shared<Add>(get_weak(), l.name, l.inputs[0], l.inputs[1]));
                break;
            case kRelu:
                alias_output(l.outputs[0], l.inputs[0]);
                layers.push_back(std::make_shared<Relu>(get_weak(), l.name, l.inputs[0]));
                break;
            case kMaxPool:
            case kAvePool:
                new_output(l.outputs[0]);
                if (l.type == kMaxPool)
                    layers.push_back(std::make_shared<MaxPool>(get_weak(), l.name, l.inputs[0], l.outputs[0], l.kernel_shape[0],
                                                               l.kernel_shape[1], l.pad_h, l.pad_w, l.stride_h, l.stride_w));
                else
                    layers.push_back(std::make_shared<AvePool>(get_weak(), l.name, l.inputs[0], l.outputs[0], l.kernel_shape[0],
                                                               l.kernel_shape[1], l.pad_h, l.pad_w, l.stride_h, l.stride_w));
                break;
            case kPRelu:
                alias_output(l.outputs[0], l.inputs[0]);
                layers.push_back(std::make_shared<PRelu>(get_weak(), l.name, l.inputs[0], l.slope));
                break;
            case kConcat:
                new_output(l.outputs[0]);
                layers.push_back(std::make_shared<Concat>(get_weak(), l.name, l.inputs[0], l.inputs[1], l.outputs[0]));
                break;
            case kSplit: {  // dabnn/net.cpp:245-250: the outputs take the input's type and image count
                const int images = blob(l.inputs[0])->n;
                new_output(l.outputs[0], DataType::Bit, images);
                new_output(l.outputs[1], DataType::Bit, images);
                layers.push_back(std::make_shared<Split>(get_weak(), l.name, l.inputs[0], l.outputs[0], l.outputs[1]));
                break;
            }
            case kShuffle:
                alias_output(l.outputs[0], l.inputs[0]);
                layers.push_back(std::make_shared<Shuffle>(get_weak(), l.name, l.inputs[0]));
                break;
            default:
                throw std::runtime_error(std::string("Not supported op ") + layer_type_name(l.type));
        }
    }
    if (optimize) fuse_binconv_epilogues();
    // an in-place layer on the input blob would write into a caller's buffer that is read in place
    copy_input_ = layers_write_input();
    hip_check(hipStreamSynchronize(static_cast<hipStream_t>(stream_)), "hipStreamSynchronize");
    prepared_ = true;
}

// Blobs a layer reads and writes (in-place layers do both).
static void layer_io(const std::shared_ptr<Layer> &l, std::vector<const Mat *> &reads, std::vector<const Mat *> &writes) {
    reads.clear(), writes.clear();
    if (auto bc = std::dynamic_pointer_cast<BinConv>(l)) {
        reads = {bc->input_mat.get()};
        writes = {bc->output_mat.get(), bc->binarized_mat.get(), bc->col_mat.get()};
    } else if (auto fc = std::dynamic_pointer_cast<FloatConv>(l)) {
        reads = {fc->fused_pool_input ? fc->fused_pool_input.get() : fc->input_mat.get()};
        writes = {fc->output_mat ? fc->output_mat.get() : fc->fused_maxpool_out.get()};
        if (fc->fused_maxpool_sign) writes.push_back(fc->fused_maxpool_sign.get());
        if (fc->fused_pool_input && fc->input_mat->dev) writes.push_back(fc->input_mat.get());  // the pooled blob, a side product
    } else if (auto af = std::dynamic_pointer_cast<Affine>(l)) {
        reads = writes = {af->data_mat.get()};
    } else if (auto ad = std::dynamic_pointer_cast<Add>(l)) {
        reads = {ad->input1_mat.get(), ad->input2_mat.get()};
        writes = {ad->input1_mat.get()};
    } else if (auto re = std::dynamic_pointer_cast<Relu>(l)) {
        reads = writes = {re->data_mat.get()};
    } else if (auto pr = std::dynamic_pointer_cast<PRelu>(l)) {
        reads = writes = {pr->data_mat.get()};
    } else if (auto cc = std::dynamic_pointer_cast<Concat>(l)) {
        reads = {cc->input1_mat.get(), cc->input2_mat.get()};
        writes = {cc->output_mat.get()};
    } else if (auto ap = std::dynamic_pointer_cast<AvePool>(l)) {
        reads = {ap->input_mat.get()};
        writes = {ap->output_mat.get()};
    } else if (auto mp = std::dynamic_pointer_cast<MaxPool>(l)) {
        reads = {mp->input_mat.get()};
        writes = {mp->output_mat.get()};
    } else if (auto sp = std::dynamic_pointer_cast<Split>(l)) {
        reads = {sp->input_mat.get()};
        writes = {sp->output_mat1.get(), sp->output_mat2.get()};
    } else if (auto sh = std::dynamic_pointer_cast<Shuffle>(l)) {
        reads = writes = {sh->data_mat.get()};
    }
}

bool Net::layers_write_input() {
    std::vector<const Mat *> rd, wr;
    const Mat *in = blob(input_name_).get();
    for (const auto &l : layers) {
        layer_io(l, rd, wr);
        for (const Mat *m : wr)
            if (m == in) return true;
    }
    return false;
}

static bool contains(const std::vector<const Mat *> &v, const Mat *m) {
    for (const Mat *x : v)
        if (x == m) return true;
    return false;
}

// Three rewrites of the layer list; blob names and contents after run() are unchanged, because the in-place layers
// wrote into the convolution's output blob anyway.
//  1. In a down-sampling block the converter emits BinConv, Affine, [AvePool, FpConv2D, Affine], Add: the shortcut
//     branch in brackets neither reads nor writes the BinConv's blobs, so BinConv and Affine move behind it, next to
//     their Add.
//  2. BinConv -> Affine (-> Add) on the same blob becomes one pass of the direct kernel, FloatConv -> Affine (-> Relu)
//     one pass of the float convolution.
//  3. When the blob such a fused BinConv completes is the input of a later direct BinConv, the pass also writes that
//     layer's packed input and the later layer skips its pack_mat.
//  4. AvePool 2x2 stride 2 -> 1x1 FloatConv (the shortcut branch of a down-sampling block), the convolution being
//     the only reader of the pooled blob, becomes one launch that does not write that blob: it leaves the net
//     (get_blob says why).  With eight pooled pixels or fewer the blob stays and is written.
//  5. FloatConv (-> Affine -> Relu) -> MaxPool 3x3 stride 2 pad 1, the pool being the only reader of the convolution's
//     blob (the stem), becomes one pass that never writes that blob when the library says the pass pays for these
//     shapes; the blob leaves the net (get_blob says why) and its memory, four times the pooled blob's, is freed.
void Net::fuse_binconv_epilogues() {
    std::vector<const Mat *> rd, wr;
    for (size_t i = 0; i + 2 < layers.size(); ++i) {
        auto bc = std::dynamic_pointer_cast<BinConv>(layers[i]);
        auto af = std::dynamic_pointer_cast<Affine>(layers[i + 1]);
        if (!bc || !af || af->data_mat != bc->output_mat) continue;
        size_t j = i + 2;
        bool movable = true;
        for (; j < layers.size(); ++j) {
            layer_io(layers[j], rd, wr);
            if (contains(rd, bc->output_mat.get()) || contains(wr, bc->output_mat.get())) break;
            // the branch must not disturb what the BinConv reads, nor use its scratch
            if (contains(wr, bc->input_mat.get()) || contains(rd, bc->binarized_mat.get()) ||
                contains(wr, bc->binarized_mat.get()) || rd.empty())
                movable = false;
        }
        auto ad = j < layers.size() ? std::dynamic_pointer_cast<Add>(layers[j]) : nullptr;
        if (!movable || j == i + 2 || !ad || ad->input1_mat != bc->output_mat || ad->input2_mat == bc->output_mat) continue;
        std::rotate(layers.begin() + i, layers.begin() + i + 2, layers.begin() + j);  // [bc, af, branch...] -> [branch..., bc, af]
        i = j;  // continue behind the Add
    }

    std::vector<std::shared_ptr<Layer>> out;
    for (size_t i = 0; i < layers.size(); ++i) {
        auto bc = std::dynamic_pointer_cast<BinConv>(layers[i]);
        auto af = i + 1 < layers.size() ? std::dynamic_pointer_cast<Affine>(layers[i + 1]) : nullptr;
        // (1024 input channels: the direct kernel counts them in two passes and has no fused epilogue)
        if (bc && af && bc->method() == BinConv::DIRECT_CONV && bc->input_mat->elem_c <= 512 && af->data_mat == bc->output_mat &&
            bc->output_mat->c % 4 == 0) {
            bc->fused_a = af->a_mat;
            bc->fused_b = af->b_mat;
            size_t skip = 1;
            auto ad = i + 2 < layers.size() ? std::dynamic_pointer_cast<Add>(layers[i + 2]) : nullptr;
            if (ad && ad->input1_mat == bc->output_mat && ad->input2_mat != bc->output_mat) {
                bc->fused_shortcut = ad->input2_mat;
                skip = 2;
            }
            out.push_back(bc);
            i += skip;
        } else if (auto fc = std::dynamic_pointer_cast<FloatConv>(layers[i])) {
            // FloatConv -> Affine (-> Relu), all on the convolution's output blob
            size_t skip = 0;
            if (af && af->data_mat == fc->output_mat) {
                fc->fused_a = af->a_mat;
                fc->fused_b = af->b_mat;
                skip = 1;
            }
            auto re = i + skip + 1 < layers.size() ? std::dynamic_pointer_cast<Relu>(layers[i + skip + 1]) : nullptr;
            if (re && re->data_mat == fc->output_mat) {
                fc->fused_relu = true;
                ++skip;
            }
            out.push_back(fc);
            i += skip;
        } else {
            out.push_back(layers[i]);
        }
    }
    layers.swap(out);

    // the same for a MaxPool whose output a direct BinConv packs (the first block of a Bi-Real net)
    for (size_t i = 0; i < layers.size(); ++i) {
        auto pool = std::dynamic_pointer_cast<MaxPool>(layers[i]);
        if (!pool || pool->output_mat->c % 64 != 0) continue;
        for (size_t j = i + 1; j < layers.size(); ++j) {
            auto consumer = std::dynamic_pointer_cast<BinConv>(layers[j]);
            if (consumer && consumer->input_mat == pool->output_mat) {
                if (consumer->method() == BinConv::DIRECT_CONV && !consumer->input_prepacked) {
                    pool->fused_sign_out = consumer->binarized_mat;
                    consumer->input_prepacked = true;
                }
                break;
            }
            layer_io(layers[j], rd, wr);
            if (contains(wr, pool->output_mat.get())) break;
        }
    }
    for (size_t i = 0; i < layers.size(); ++i) {
        auto producer = std::dynamic_pointer_cast<BinConv>(layers[i]);
        if (!producer || !producer->fused_a || producer->output_mat->c % 64 != 0) continue;
        // not with 512 input channels: sign bits need work items of 8 output channels, four units there, and the
        // coarser split costs more than the separate pack_mat it saves (measured at batch 64 and 256) -- unless the
        // problem is small enough for the kernel whose work items are 8 channels anyway, or of the size that the
        // row-split kernel takes (its store pass writes the bits at no extra pass)
        if (producer->input_mat->elem_c >= 512) {
            const int64_t pixels = (int64_t)producer->output_mat->n * producer->output_mat->h * producer->output_mat->w;
            if (!dab_bconv3x3_splits_depth(pixels, producer->input_mat->elem_c, producer->output_mat->c) &&
                dab_bconv3x3_epilogue_build(pixels, producer->input_mat->elem_c, producer->output_mat->c, producer->stride_h, 1) != 3)
                continue;
        }
        for (size_t j = i + 1; j < layers.size(); ++j) {
            auto consumer = std::dynamic_pointer_cast<BinConv>(layers[j]);
            if (consumer && consumer->input_mat == producer->output_mat) {
                if (consumer->method() == BinConv::DIRECT_CONV) {
                    producer->fused_sign_out = consumer->binarized_mat;
                    consumer->input_prepacked = true;
                }
                break;
            }
            layer_io(layers[j], rd, wr);
            if (contains(wr, producer->output_mat.get())) break;  // the blob changes again before anyone packs it
        }
    }

    for (size_t i = 0; i + 1 < layers.size(); ++i) {
        auto pool = std::dynamic_pointer_cast<AvePool>(layers[i]);
        if (!pool || pool->pad_h != 0 || pool->pad_w != 0 || pool->input_mat->c % 4 != 0) continue;
        const bool two_by_two = pool->kernel_h == 2 && pool->kernel_w == 2 && pool->stride_h == 2 && pool->stride_w == 2 &&
                                pool->input_mat->h >= 2 && pool->input_mat->w >= 2;
        // one window over the whole image (the pool before a classifier); whether the one-launch form covers the shapes
        // is asked below, when the convolution is known
        const bool global = !two_by_two && pool->kernel_h == pool->input_mat->h && pool->kernel_w == pool->input_mat->w;
        if (!two_by_two && !global) continue;
        // the one reader of the pooled blob must be a 1x1 FloatConv, with nothing in between that rewrites the pool's input
        size_t j = i + 1;
        bool ok = true;
        for (; j < layers.size(); ++j) {
            layer_io(layers[j], rd, wr);
            if (contains(rd, pool->output_mat.get())) break;
            if (contains(wr, pool->input_mat.get()) || contains(wr, pool->output_mat.get())) ok = false;
        }
        auto fc = j < layers.size() ? std::dynamic_pointer_cast<FloatConv>(layers[j]) : nullptr;
        if (!ok || !fc || fc->input_mat != pool->output_mat || fc->weight_mat->h != 1 || fc->weight_mat->w != 1 ||
            fc->pad_h != 0 || fc->pad_w != 0 || fc->stride_h != 1 || fc->stride_w != 1 || fc->dilation != 1)
            continue;
        for (size_t k = j + 1; k < layers.size() && ok; ++k) {
            layer_io(layers[k], rd, wr);
            if (contains(rd, pool->output_mat.get())) ok = false;  // someone else wants the pooled blob at its own time
        }
        if (!ok) continue;
        if (global && !dab_global_ave_pool_fconv1x1_takes(pool->input_mat->n, pool->input_mat->h, pool->input_mat->w,
                                                          pool->input_mat->c, fc->output_mat->c))
            continue;
        fc->fused_pool_input = pool->input_mat;
        fc->fused_pool_global = global;
        // Nobody but this convolution reads the pooled blob, so the 2x2 form does not write it: the blob leaves the
        // net (get_blob says why) and a Mat without memory keeps its shape for the layer.  Eight pooled pixels or
        // fewer run as the two launches and keep the blob.
        const Mat &pooled = *pool->output_mat;
        if (!global && (long long)pooled.n * pooled.h * pooled.w > 8) {
            for (auto it = mat_map_.begin(); it != mat_map_.end();) {
                if (it->second == pool->output_mat) {
                    elided_[it->first] = "the AvePool runs inside the convolution that reads it";
                    it = mat_map_.erase(it);
                } else {
                    ++it;
                }
            }
            fc->input_mat = std::make_shared<Mat>(pooled.n, pooled.h, pooled.w, pooled.c, nullptr, DataType::Float);
        }
        layers.erase(layers.begin() + i);
        --i;
    }

    for (size_t i = 0; i + 1 < layers.size(); ++i) {
        auto fc = std::dynamic_pointer_cast<FloatConv>(layers[i]);
        auto pool = std::dynamic_pointer_cast<MaxPool>(layers[i + 1]);
        if (!fc || !pool || fc->fused_pool_input || pool->input_mat != fc->output_mat || pool->kernel_h != 3 ||
            pool->kernel_w != 3 || pool->stride_h != 2 || pool->stride_w != 2 || pool->pad_h != 1 || pool->pad_w != 1)
            continue;
        bool only_reader = true;
        for (size_t j = 0; j < layers.size() && only_reader; ++j) {
            if (j == i || j == i + 1) continue;
            layer_io(layers[j], rd, wr);
            if (contains(rd, fc->output_mat.get()) || contains(wr, fc->output_mat.get())) only_reader = false;
        }
        const Mat &in = *fc->input_mat;
        const Mat &wt = *fc->weight_mat;
        if (!only_reader || !dab_fconv_maxpool_pays(in.n, in.h, in.w, in.c, wt.h, wt.w, fc->pad_h, fc->pad_w, fc->stride_h,
                                                    fc->stride_w, fc->dilation, fc->dilation, wt.n))
            continue;
        const int64_t carry = dab_fconv_maxpool_carry_floats(in.n, in.h, in.w, in.c, wt.h, wt.w, fc->pad_h, fc->pad_w,
                                                             fc->stride_h, fc->stride_w, fc->dilation, fc->dilation, wt.n);
        fc->fused_maxpool_out = pool->output_mat;
        fc->fused_maxpool_sign = pool->fused_sign_out;
        fc->fused_maxpool_carry = std::make_shared<Mat>((size_t)carry, DataType::Float, fc->name_ + "_carry");
        for (auto it = mat_map_.begin(); it != mat_map_.end();) {
            if (it->second == fc->output_mat) {
                elided_[it->first] = "the convolution and the MaxPool behind it run as one pass";
                it = mat_map_.erase(it);
            } else {
                ++it;
            }
        }
        fc->output_mat.reset();
        layers.erase(layers.begin() + i + 1);
    }
}

void Net::run(const void *host_input) {
    BNN_ASSERT(prepared_, "run before read");
    BNN_ASSERT(host_input != nullptr, "run: null input");
    bind_input(nullptr);
    auto in = blob(input_name_);
    hip_check(hipMemcpyAsync(in->dev, host_input, in->bytes(), hipMemcpyHostToDevice, static_cast<hipStream_t>(stream_)),
              "hipMemcpyAsync");
    launch_layers();
}

void Net::run_device(const void *device_input) {
    BNN_ASSERT(prepared_, "run before read");
    bind_input(device_input);
    launch_layers();
}

// Points the input blob at the memory this run reads: the caller's device buffer in place, or the blob's own
// allocation (host inputs, unaligned buffers, callers whose buffers keep changing), filled here from device_input.
void Net::bind_input(const void *device_input) {
    auto in = blob(input_name_);
    const bool in_place = device_input != nullptr && !copy_input_ && reinterpret_cast<uintptr_t>(device_input) % 256 == 0;
    void *want = in_place ? const_cast<void *>(device_input) : input_own_dev_;
    if (graph_exec_ && graph_input_ != want) {
        // the graph's kernels hold the address they were captured with
        if (in_place && ++input_rebinds_ >= 3) {
            copy_input_ = true;
            want = input_own_dev_;
        }
        if (graph_input_ != want) {
            std::lock_guard<std::mutex> lock(capture_mutex());
            (void)hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec_));
            graph_exec_ = nullptr;
        }
    }
    in->dev = want;
    if (device_input != nullptr && want == input_own_dev_ && device_input != input_own_dev_)
        hip_check(hipMemcpyAsync(in->dev, device_input, in->bytes(), hipMemcpyDeviceToDevice, static_cast<hipStream_t>(stream_)),
                  "hipMemcpyAsync");
}

void Net::launch_layers() {
    BNN_ASSERT(!(strict && !run_fconv), "fconv must be run in strict mode");
    hipStream_t s = static_cast<hipStream_t>(stream_);
    if (profile || !use_graph) {
        for (const auto &layer : layers) layer->forward();
    } else if (graph_exec_) {
        hip_check(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec_), s), "hipGraphLaunch");
    } else if (runs_ >= 2) {
        // capture the kernels of one forward pass; nothing in the layers allocates, synchronises or memsets
        std::lock_guard<std::mutex> lock(capture_mutex());
        hipGraph_t graph = nullptr;
        hip_check(hipStreamBeginCapture(s, hipStreamCaptureModeThreadLocal), "hipStreamBeginCapture");
        try {
            for (const auto &layer : layers) layer->forward();
        } catch (...) {
            (void)hipStreamEndCapture(s, &graph);
            if (graph) (void)hipGraphDestroy(graph);
            throw;
        }
        hip_check(hipStreamEndCapture(s, &graph), "hipStreamEndCapture");
        hipGraphExec_t exec = nullptr;
        hip_check(hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0), "hipGraphInstantiate");
        (void)hipGraphDestroy(graph);
        graph_exec_ = exec;
        graph_input_ = blob(input_name_)->dev;
        hip_check(hipGraphLaunch(exec, s), "hipGraphLaunch");
    } else {
        for (const auto &layer : layers) layer->forward();
    }
    ++runs_;
    hip_check(hipStreamSynchronize(s), "hipStreamSynchronize");
    for (const auto &kv : mat_map_) kv.second->mark_device_written();  // host mirrors show the previous run
}

std::vector<std::string> Net::layer_descriptions() const {
    std::vector<std::string> out;
    for (const auto &l : layers) out.push_back(l->to_str());
    return out;
}

std::string Net::time_report() const {
    std::stringstream ss;
    double total = 0;
    for (const auto &kv : layer_time_) total += kv.second;
    for (const auto &kv : layer_time_) ss << kv.first << ": " << kv.second << "ms\n";
    ss << "total: " << total << "ms\n";
    return ss.str();
}

}  // namespace bnn
