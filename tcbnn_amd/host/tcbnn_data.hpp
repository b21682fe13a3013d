// Dataset readers and the accuracy check of the reference's host side (data.h:36-119,
// data.cpp, utility.h:198-233), host-only C++ with no GPU dependency: the same function names,
// argument meaning, output layouts and normalisation arithmetic, so that a driver written
// against the reference reads its evaluation batch unchanged.
//
//   read_MNIST_raw / read_MNIST_normalized        idx3-ubyte images + idx1-ubyte labels
//   read_CIFAR10_raw / read_CIFAR10_normalized    the binary batches <label><R 1024><G 1024><B 1024>
//   read_ImageNet_normalized                      "<file>,<label>" list; resize to a 256 short side
//                                                 with the reference's bilinear routine, centre crop
//                                                 224x224, normalise, CHW
//   validate_prediction                           top-1 / top-5 of a [batch][categories] logit array
//
// Differences, all on the error path or the decoder: a file that cannot be opened or ends early
// is reported and exits with status 1 (the reference checks only the open); the ImageNet reader
// decodes binary PPM (P6) files, because libjpeg is not part of this build, and the resize writes
// only the pixels of the scaled image (the reference's loop also writes one element past each
// row and one row past the end, none of which the centre crop reads).
#pragma once

#include <math.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <string>
#include <vector>

typedef unsigned char uchar;

namespace tcbnn_data {

inline void need(const void* p, const char* what) {
    if (p == NULL) {
        fprintf(stderr, "NULL %s pointer in reading a dataset.\n", what);
        exit(1);
    }
}

inline FILE* open_or_die(const std::string& path, const char* what) {
    FILE* f = fopen(path.c_str(), "rb");
    if (f == NULL) {
        fprintf(stderr, "Error in reading %s file '%s'.\n", what, path.c_str());
        exit(1);
    }
    return f;
}

inline void read_or_die(FILE* f, void* dst, size_t n, const std::string& path) {
    if (n != 0 && fread(dst, 1, n, f) != n) {
        fprintf(stderr, "File '%s' ended early.\n", path.c_str());
        exit(1);
    }
}

// big-endian 32-bit header field of the idx formats (ReverseInt, data.cpp:18-26)
inline int read_be32(FILE* f, const std::string& path) {
    uchar b[4];
    read_or_die(f, b, 4, path);
    return (int)(((unsigned)b[0] << 24) | ((unsigned)b[1] << 16) | ((unsigned)b[2] << 8) | (unsigned)b[3]);
}

// The first `batch` images of an idx3 file as bytes, and the first `batch` labels of an idx1 file.
inline void read_mnist_bytes(const std::string& filename, const std::string& labelname, uchar* pixels,
                             unsigned* labels, unsigned batch) {
    const size_t px = 28 * 28;
    FILE* f = open_or_die(filename, "MNIST image");
    for (int i = 0; i < 4; ++i) (void)read_be32(f, filename);  // magic, count, rows, cols: not checked (data.cpp:57-64)
    read_or_die(f, pixels, (size_t)batch * px, filename);
    fclose(f);
    FILE* lf = open_or_die(labelname, "MNIST label");
    for (int i = 0; i < 2; ++i) (void)read_be32(lf, labelname);
    std::vector<uchar> lab(batch);
    read_or_die(lf, lab.data(), batch, labelname);
    fclose(lf);
    for (unsigned i = 0; i < batch; ++i) labels[i] = lab[i];
}

}  // namespace tcbnn_data

// data.cpp:28-110: [batch][28][28] bytes
inline void read_MNIST_raw(std::string filename, std::string labelname, uchar* images, unsigned* labels,
                           const unsigned batch) {
    tcbnn_data::need(images, "images");
    tcbnn_data::need(labels, "labels");
    tcbnn_data::read_mnist_bytes(filename, labelname, images, labels, batch);
}

// data.cpp:112-194: [batch][1][28][28] floats, (v/255 - 0.1307) / 0.3081
inline void read_MNIST_normalized(std::string filename, std::string labelname, float* images, unsigned* labels,
                                  const unsigned batch) {
    tcbnn_data::need(images, "images");
    tcbnn_data::need(labels, "labels");
    std::vector<uchar> raw((size_t)batch * 28 * 28);
    tcbnn_data::read_mnist_bytes(filename, labelname, raw.data(), labels, batch);
    for (size_t i = 0; i < raw.size(); ++i) images[i] = (((float)raw[i] / 255.f) - 0.1307f) / 0.3081f;
}

// data.cpp:198-245: [batch][32][32] words, byte c of a word = channel c, the fourth byte 0
inline void read_CIFAR10_raw(std::string filename, unsigned* images, unsigned* labels, const unsigned batch) {
    tcbnn_data::need(images, "images");
    tcbnn_data::need(labels, "labels");
    memset(images, 0, (size_t)batch * 32 * 32 * sizeof(unsigned));
    uchar* ui = reinterpret_cast<uchar*>(images);
    FILE* f = tcbnn_data::open_or_die(filename, "Cifar-10 bin");
    std::vector<uchar> rec(1 + 3 * 1024);
    for (unsigned l = 0; l < batch; ++l) {
        tcbnn_data::read_or_die(f, rec.data(), rec.size(), filename);
        labels[l] = rec[0];
        for (int c = 0; c < 3; ++c)
            for (int p = 0; p < 1024; ++p) ui[((size_t)l * 1024 + p) * 4 + c] = rec[1 + c * 1024 + p];
    }
    fclose(f);
}

// data.cpp:248-316: [batch][3][32][32] floats, (v/255 - mean_c) / std_c
inline void read_CIFAR10_normalized(std::string filename, float* images, unsigned* labels, const unsigned batch) {
    tcbnn_data::need(images, "images");
    tcbnn_data::need(labels, "labels");
    static const float mean[3] = {0.4914f, 0.4822f, 0.4465f};
    static const float stdv[3] = {0.2470f, 0.2435f, 0.2616f};
    FILE* f = tcbnn_data::open_or_die(filename, "Cifar-10 bin");
    std::vector<uchar> rec(1 + 3 * 1024);
    for (unsigned l = 0; l < batch; ++l) {
        tcbnn_data::read_or_die(f, rec.data(), rec.size(), filename);
        labels[l] = rec[0];
        for (int c = 0; c < 3; ++c)
            for (int p = 0; p < 1024; ++p)
                images[((size_t)l * 3 + c) * 1024 + p] = ((float)rec[1 + c * 1024 + p] / 255.0f - mean[c]) / stdv[c];
    }
    fclose(f);
}

namespace tcbnn_data {

// Resize (short side to 256, bilinear on bytes, truncating), centre crop to out_h x out_w,
// normalise: read_normalized_jpeg after the decode (data.cpp:478-552) with scale_transform
// (data.cpp:407-431).  `hwc` is the decoded image, 3 bytes per pixel.
inline void imagenet_preprocess(const uchar* hwc, int org_h, int org_w, float* fdata, int out_h, int out_w) {
    std::vector<uchar> chw((size_t)3 * org_h * org_w);
    for (int h = 0; h < org_h; ++h)
        for (int w = 0; w < org_w; ++w)
            for (int c = 0; c < 3; ++c) chw[((size_t)c * org_h + h) * org_w + w] = hwc[((size_t)h * org_w + w) * 3 + c];
    const float scale = 256.0f / std::min((unsigned long)org_w, (unsigned long)org_h);
    int sh, sw;
    if (org_w < org_h) {
        sw = 256;
        sh = int(scale * org_h);
    } else {
        sh = 256;
        sw = int(scale * org_w);
    }
    if (sh < out_h || sw < out_w) {
        fprintf(stderr, "image %dx%d is too small for a %dx%d crop.\n", org_h, org_w, out_h, out_w);
        exit(1);
    }
    std::vector<uchar> scaled((size_t)3 * sh * sw);
    for (int y = 0; y < sh; ++y)
        for (int x = 0; x < sw; ++x) {
            const float gx = x / (float)(sw) * (org_w - 1);
            const float gy = y / (float)(sh) * (org_h - 1);
            const int gxi = (int)gx, gyi = (int)gy;
            for (int c = 0; c < 3; ++c) {
                const uchar* s = &chw[(size_t)c * org_w * org_h];
                const float c00 = (float)s[(size_t)gyi * org_w + gxi];
                const float c10 = (float)s[(size_t)gyi * org_w + gxi + 1];
                const float c01 = (float)s[(size_t)(gyi + 1) * org_w + gxi];
                const float c11 = (float)s[(size_t)(gyi + 1) * org_w + gxi + 1];
                const float tx = gx - gxi, ty = gy - gyi;
                const float top = c00 + (c10 - c00) * tx;
                const float bot = c01 + (c11 - c01) * tx;
                scaled[((size_t)c * sh + y) * sw + x] = (uchar)(top + (bot - top) * ty);
            }
        }
    static const float mul[3] = {4.3668f, 4.4643f, 4.4444f};
    static const float sub[3] = {2.1179f, 2.0357f, 1.8044f};
    for (int h = 0; h < out_h; ++h)
        for (int w = 0; w < out_w; ++w) {
            const int mh = h + (sh - out_h) / 2, mw = w + (sw - out_w) / 2;
            for (int c = 0; c < 3; ++c)
                fdata[((size_t)c * out_h + h) * out_w + w] =
                    ((float)scaled[((size_t)c * sh + mh) * sw + mw] / 255.0f) * mul[c] - sub[c];
        }
}

// A binary PPM (P6, maxval 255): fills hwc, returns height and width.
inline void read_ppm(const std::string& path, std::vector<uchar>* hwc, int* h, int* w) {
    FILE* f = open_or_die(path, "PPM image");
    int maxval = 0;
    char magic[3] = {0, 0, 0};
    if (fscanf(f, "%2s", magic) != 1 || strcmp(magic, "P6") != 0) {
        fprintf(stderr, "'%s' is not a binary PPM (P6) file.\n", path.c_str());
        exit(1);
    }
    int vals[3], got = 0;
    while (got < 3) {
        int ch = fgetc(f);
        if (ch == '#') {
            while (ch != '\n' && ch != EOF) ch = fgetc(f);
        } else if (ch == EOF) {
            break;
        } else if (ch > ' ') {
            ungetc(ch, f);
            if (fscanf(f, "%d", &vals[got]) != 1) break;
            ++got;
        }
    }
    if (got == 3) {
        *w = vals[0];
        *h = vals[1];
        maxval = vals[2];
    }
    if (got != 3 || maxval != 255 || *w <= 0 || *h <= 0) {
        fprintf(stderr, "'%s': unsupported PPM header.\n", path.c_str());
        exit(1);
    }
    fgetc(f);  // the single white-space byte after maxval
    hwc->resize((size_t)3 * *w * *h);
    read_or_die(f, hwc->data(), hwc->size(), path);
    fclose(f);
}

}  // namespace tcbnn_data

// data.cpp:554-593: [batch][3][224][224] floats; each line of the list is "<image file>,<label>"
inline void read_ImageNet_normalized(const char* descfilename, float* images, unsigned* labels, int batch) {
    tcbnn_data::need(images, "images");
    tcbnn_data::need(labels, "labels");
    FILE* desc = fopen(descfilename, "r");
    if (desc == NULL) {
        fprintf(stderr, "Error reading Imagenet Description File '%s'.\n", descfilename);
        exit(1);
    }
    char filename[1024];
    std::vector<uchar> hwc;
    for (int i = 0; i < batch; ++i) {
        unsigned tag = 0;
        if (fscanf(desc, " %1023[^,\n],", filename) != 1 || fscanf(desc, "%u", &tag) != 1) {
            fprintf(stderr, "Imagenet Description File '%s' ended after %d of %d entries.\n", descfilename, i, batch);
            exit(1);
        }
        labels[i] = tag;
        int h = 0, w = 0;
        tcbnn_data::read_ppm(filename, &hwc, &h, &w);
        tcbnn_data::imagenet_preprocess(hwc.data(), h, w, images + (size_t)i * 3 * 224 * 224, 224, 224);
    }
    fclose(desc);
}

// What validate_prediction counted.
struct PredictionScore {
    int top1, top5, batch;
};

// utility.h:198-233, including how it ranks: one pass over the categories keeps a best value and four
// runner-up slots, every slot starting at the score of category 0 with position 0; a value that beats
// the best replaces it WITHOUT moving the old best down, otherwise the first slot it beats takes it.
// The slots therefore hold some large values, not always the five largest, and "top-5" is the
// reference's count, not the textbook one.  Prints the same report; also returns the counts.
inline PredictionScore score_prediction(const float* prediction, const unsigned* labels, unsigned categories,
                                        unsigned batch, std::vector<int>* top1_positions = NULL) {
    PredictionScore sc = {0, 0, (int)batch};
    for (unsigned i = 0; i < batch; ++i) {
        const float* p = prediction + (size_t)i * categories;
        float best[5] = {p[0], p[0], p[0], p[0], p[0]};
        int pos[5] = {0, 0, 0, 0, 0};
        for (unsigned j = 0; j < categories; ++j)
            for (int k = 0; k < 5; ++k)
                if (p[j] > best[k]) {
                    best[k] = p[j];
                    pos[k] = (int)j;
                    break;
                }
        if (top1_positions) top1_positions->push_back(pos[0]);
        if ((unsigned)pos[0] == labels[i]) sc.top1 += 1;
        for (int k = 0; k < 5; ++k)
            if ((unsigned)pos[k] == labels[i]) {
                sc.top5 += 1;
                break;
            }
    }
    return sc;
}

inline PredictionScore validate_prediction(float* prediction, unsigned* labels, const unsigned categories,
                                           const unsigned batch) {
    printf("======Label======\n");
    for (unsigned i = 0; i < batch; i++) printf("%u ", labels[i]);
    printf("\n=====Predict=======\n");
    std::vector<int> pos;
    const PredictionScore sc = score_prediction(prediction, labels, categories, batch, &pos);
    for (unsigned i = 0; i < batch; i++) printf("%d ", pos[i]);
    printf("\n=====Batch Accuracy:%d=======\n", batch);
    printf("Top-1:%f%%\n", float(sc.top1) / batch * 100);
    printf("Top-5:%f%%\n", float(sc.top5) / batch * 100);
    return sc;
}
