// Host-only companion of the network drivers: reads an evaluation batch with the dataset readers
// (data.h:36-119 of the reference) and writes it as the raw float32 file the drivers take with
// --input, plus the labels as raw uint32; or scores a logits file the drivers wrote with --out
// (validate_prediction, utility.h:198-233).  No GPU and no HIP runtime involved.
#include <stdint.h>

#include "../host/tcbnn_data.hpp"

static void write_raw(const char* path, const void* data, size_t bytes) {
    FILE* f = fopen(path, "wb");
    if (f == NULL || fwrite(data, 1, bytes, f) != bytes) {
        fprintf(stderr, "cannot write %s\n", path);
        exit(1);
    }
    fclose(f);
}

static std::vector<char> read_raw(const char* path, size_t bytes) {
    std::vector<char> v(bytes);
    FILE* f = tcbnn_data::open_or_die(path, "raw");
    tcbnn_data::read_or_die(f, v.data(), bytes, path);
    fclose(f);
    return v;
}

int main(int argc, char** argv) {
    const char* usage =
        "read_dataset mnist <images-idx3> <labels-idx1> <batch> <out.f32> <labels.u32>\n"
        "read_dataset cifar10 <batch.bin> <batch> <out.f32> <labels.u32>\n"
        "read_dataset imagenet <list: file.ppm,label per line> <batch> <out.f32> <labels.u32>\n"
        "read_dataset validate <logits.f32> <labels.u32> <categories> <batch>\n";
    const std::string mode = argc > 1 ? argv[1] : "";
    if (mode == "mnist" && argc == 7) {
        const unsigned batch = (unsigned)atoi(argv[4]);
        std::vector<float> img((size_t)batch * 28 * 28);
        std::vector<unsigned> lab(batch);
        read_MNIST_normalized(argv[2], argv[3], img.data(), lab.data(), batch);
        write_raw(argv[5], img.data(), img.size() * sizeof(float));
        write_raw(argv[6], lab.data(), lab.size() * sizeof(unsigned));
    } else if (mode == "cifar10" && argc == 6) {
        const unsigned batch = (unsigned)atoi(argv[3]);
        std::vector<float> img((size_t)batch * 3 * 32 * 32);
        std::vector<unsigned> lab(batch);
        read_CIFAR10_normalized(argv[2], img.data(), lab.data(), batch);
        write_raw(argv[4], img.data(), img.size() * sizeof(float));
        write_raw(argv[5], lab.data(), lab.size() * sizeof(unsigned));
    } else if (mode == "imagenet" && argc == 6) {
        const int batch = atoi(argv[3]);
        std::vector<float> img((size_t)batch * 3 * 224 * 224);
        std::vector<unsigned> lab(batch);
        read_ImageNet_normalized(argv[2], img.data(), lab.data(), batch);
        write_raw(argv[4], img.data(), img.size() * sizeof(float));
        write_raw(argv[5], lab.data(), lab.size() * sizeof(unsigned));
    } else if (mode == "validate" && argc == 6) {
        const unsigned categories = (unsigned)atoi(argv[4]), batch = (unsigned)atoi(argv[5]);
        std::vector<char> logits = read_raw(argv[2], (size_t)batch * categories * sizeof(float));
        std::vector<char> labels = read_raw(argv[3], (size_t)batch * sizeof(unsigned));
        validate_prediction(reinterpret_cast<float*>(logits.data()), reinterpret_cast<unsigned*>(labels.data()),
                            categories, batch);
    } else {
        fputs(usage, stderr);
        return 1;
    }
    return 0;
}
