// Raw tensor files as the reference's device wrappers read and write them (test/utils/dsp/include/tensor.h:235-260):
// int32 data type id, int64 rank, rank x int64 extents, then the elements row-major. Ids used here: 1 = fp16,
// 2 = fp32 (tensor.h:26-38).
#pragma once
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

struct RawTensor {
  int32_t dtype = 0;
  std::vector<int64_t> shape;
  std::vector<unsigned char> bytes;
  int64_t count() const {
    int64_t n = 1;
    for (int64_t d : shape) n *= d;
    return n;
  }
};

inline int elem_size(int32_t dtype) { return dtype == 1 ? 2 : dtype == 2 ? 4 : 0; }

inline bool read_tensor(const std::string& path, RawTensor& t) {
  FILE* fp = std::fopen(path.c_str(), "rb");
  if (!fp) return false;
  int64_t rank = 0;
  bool ok = std::fread(&t.dtype, sizeof(int32_t), 1, fp) == 1 && std::fread(&rank, sizeof(int64_t), 1, fp) == 1 &&
            rank >= 0 && rank <= 8 && elem_size(t.dtype) > 0;
  if (ok) {
    t.shape.resize((size_t)rank);
    ok = rank == 0 || std::fread(t.shape.data(), sizeof(int64_t), (size_t)rank, fp) == (size_t)rank;
  }
  if (ok) {
    t.bytes.resize((size_t)(t.count() * elem_size(t.dtype)));
    ok = std::fread(t.bytes.data(), 1, t.bytes.size(), fp) == t.bytes.size();
  }
  std::fclose(fp);
  return ok;
}

inline bool write_tensor(const std::string& path, int32_t dtype, const std::vector<int64_t>& shape, const void* data) {
  FILE* fp = std::fopen(path.c_str(), "wb");
  if (!fp) return false;
  const int64_t rank = (int64_t)shape.size();
  int64_t n = 1;
  for (int64_t d : shape) n *= d;
  bool ok = std::fwrite(&dtype, sizeof(int32_t), 1, fp) == 1 && std::fwrite(&rank, sizeof(int64_t), 1, fp) == 1 &&
            (rank == 0 || std::fwrite(shape.data(), sizeof(int64_t), (size_t)rank, fp) == (size_t)rank) &&
            std::fwrite(data, (size_t)elem_size(dtype), (size_t)n, fp) == (size_t)n;
  std::fclose(fp);
  return ok;
}
