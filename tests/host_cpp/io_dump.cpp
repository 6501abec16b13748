// Runs the dataset readers of the C++ host mirror (tiny_dnn_hip.h) on a file and dumps what they
// return, for tests/test_io.py to compare with the compiled reference's output:
//   io_dump mnist_images <file> <scale_min> <scale_max> <x_pad> <y_pad> <out>
//   io_dump mnist_labels <file> <out>
//   io_dump cifar10 <file> <scale_min> <scale_max> <x_pad> <y_pad> <out>
//   io_dump archive <file> <format: 0 binary, 1 portable_binary> <out> <vectors of layer 0> <of layer 1> ...
//           (reads a weights archive with the mirror's reader and writes it again with its writer)
// <out>: int64 count, int64 length, then count*length float32 (images) and count int64 (labels).
// Exit status 3 and the message on stdout when the reader throws nn_error.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "tiny_dnn_hip.h"

using namespace tiny_dnn;

static void dump(const char *path, const std::vector<vec_t> &images, const std::vector<label_t> &labels) {
  FILE *f = std::fopen(path, "wb");
  if (!f) std::exit(4);
  const int64_t count = images.empty() ? static_cast<int64_t>(labels.size()) : static_cast<int64_t>(images.size());
  const int64_t len = images.empty() ? 0 : static_cast<int64_t>(images[0].size());
  std::fwrite(&count, 8, 1, f);
  std::fwrite(&len, 8, 1, f);
  for (const vec_t &v : images) std::fwrite(v.data(), 4, v.size(), f);
  for (label_t l : labels) {
    const int64_t v = static_cast<int64_t>(l);
    std::fwrite(&v, 8, 1, f);
  }
  std::fclose(f);
}

int main(int argc, char **argv) {
  if (argc < 4) return 2;
  try {
    std::vector<vec_t> images;
    std::vector<label_t> labels;
    if (argc >= 5 && !std::strcmp(argv[1], "archive")) {
      const file_format format = std::atoi(argv[3]) ? file_format::portable_binary : file_format::binary;
      std::vector<size_t> counts;
      for (int i = 5; i < argc; ++i) counts.push_back(static_cast<size_t>(std::atoi(argv[i])));
      std::ifstream is(argv[2], std::ios::binary);
      if (!is.good()) throw nn_error(std::string("failed to open:") + argv[2]);
      const std::vector<detail::archive_layer> layers = detail::read_weight_archive(is, counts, format);
      std::ofstream os(argv[4], std::ios::binary);
      detail::write_weight_archive(os, layers, format);
      for (const detail::archive_layer &l : layers) std::printf("%s ", l.type.c_str());
      std::puts("");
    } else if (!std::strcmp(argv[1], "mnist_labels")) {
      parse_mnist_labels(argv[2], &labels);
      dump(argv[3], images, labels);
    } else if (argc == 8 && !std::strcmp(argv[1], "mnist_images")) {
      parse_mnist_images(argv[2], &images, float_t(std::atof(argv[3])), float_t(std::atof(argv[4])),
                         std::atoi(argv[5]), std::atoi(argv[6]));
      dump(argv[7], images, labels);
    } else if (argc == 8 && !std::strcmp(argv[1], "cifar10")) {
      parse_cifar10(argv[2], &images, &labels, float_t(std::atof(argv[3])), float_t(std::atof(argv[4])),
                    std::atoi(argv[5]), std::atoi(argv[6]));
      dump(argv[7], images, labels);
    } else {
      return 2;
    }
  } catch (const nn_error &e) {
    std::puts(e.what());
    return 3;
  }
  return 0;
}
