// Reading and writing tensors in Tannic's file layout from the C++ front end, host or device.
//
// The reference defines the records (include/tannic/serialization.hpp:26-66: `Header`, `Metadata<Tensor>`, `headerof`,
// `metadataof`) but no I/O; this header adds it, so that a program built on the front end can load its parameters
// straight onto the device this backend drives:
//
//     Tensor w = tannic::hip::load("wq.tannic", Device());
//     tannic::hip::save(y, "out.tannic");           // a device tensor is brought to the host first
//
// A file is, in order and without padding (little endian):
//     Header            magic u32 = 0x43495245, version u8 = 1, checksum u16 = 0xABCD, nbytes u64 (everything that follows)
//     Metadata<Tensor>  dcode u8 (dcodeof, include/tannic/types.hpp:206-221), offset u64, nbytes u64 (of the data), rank u8
//     shape             rank x u64
//     data              the elements, row-major (bit-packed for booleans)
// the same image tannic_amd/serialization.py reads and writes.  Only contiguous tensors are written (repack a view
// first); a view's offset is not kept.  Damaged images throw tannic::Exception.
#pragma once

#include <cstddef>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <variant>
#include <vector>

#include "exceptions.hpp"
#include "resources.hpp"
#include "serialization.hpp"
#include "tensor.hpp"
#include "tannic_hip_adapter.hpp"

namespace tannic::hip {

// the file image of `tensor`
inline std::vector<std::byte> dumps(Tensor const& tensor) {
    if (!tensor.is_initialized()) throw Exception("dumps: the tensor has no storage");
    if (!tensor.is_contiguous()) throw Exception("dumps: only contiguous tensors are written; repack a view first");
    const Header header = headerof(tensor);
    Metadata<Tensor> metadata = metadataof(tensor);
    metadata.offset = 0;   // the data of the image starts at its beginning
    const size_t rank = tensor.rank(), data = tensor.nbytes();
    std::vector<std::byte> image(sizeof(Header) + sizeof(Metadata<Tensor>) + rank * sizeof(uint64_t) + data);
    std::byte* at = image.data();
    std::memcpy(at, &header, sizeof header);
    at += sizeof header;
    std::memcpy(at, &metadata, sizeof metadata);
    at += sizeof metadata;
    for (size_t d = 0; d < rank; ++d) {
        const uint64_t extent = tensor.shape()[d];
        std::memcpy(at, &extent, sizeof extent);
        at += sizeof extent;
    }
    if (std::holds_alternative<Device>(tensor.environment())) {
        const device_t device{std::get<Device>(tensor.environment()).id()};
        cuda::copyDeviceToHost(&device, tensor.bytes(), at, data);   // waits for the stream
    } else {
        std::memcpy(at, tensor.bytes(), data);
    }
    return image;
}

// the tensor a file image holds, placed in `environment`
inline Tensor loads(const std::byte* image, size_t size, Environment environment = Host{}) {
    if (size < sizeof(Header)) throw Exception("loads: shorter than a header");
    Header header;
    std::memcpy(&header, image, sizeof header);
    if (header.magic != MAGIC) throw Exception("loads: bad magic");
    if (header.version != 1) throw Exception("loads: unknown version");
    if (header.checksum != 0xABCD) throw Exception("loads: bad checksum");
    if (size - sizeof(Header) < header.nbytes || header.nbytes < sizeof(Metadata<Tensor>)) throw Exception("loads: truncated: the header announces more bytes than follow");
    Metadata<Tensor> metadata;
    std::memcpy(&metadata, image + sizeof(Header), sizeof metadata);
    const type dtype = dtypeof(metadata.dcode);
    if (dtype == unknown) throw Exception("loads: unknown dtype code");
    if (metadata.rank > 8) throw Exception("loads: the rank exceeds the 8 dimensions a tensor can have");
    if (header.nbytes != sizeof(Metadata<Tensor>) + metadata.rank * sizeof(uint64_t) + metadata.nbytes) throw Exception("loads: sizes in header and metadata disagree");
    if (metadata.offset != 0) throw Exception("loads: a non-zero storage offset is not supported");
    const std::byte* at = image + sizeof(Header) + sizeof(Metadata<Tensor>);
    std::vector<size_t> extents(metadata.rank);
    for (size_t d = 0; d < metadata.rank; ++d) {
        uint64_t extent;
        std::memcpy(&extent, at, sizeof extent);
        extents[d] = static_cast<size_t>(extent);
        at += sizeof extent;
    }
    Tensor host(dtype, Shape(extents.begin(), extents.end()));
    if (host.nbytes() != metadata.nbytes) throw Exception("loads: the shape does not hold the number of bytes the file gives");
    host.initialize();
    std::memcpy(host.bytes(), at, metadata.nbytes);
    if (std::holds_alternative<Host>(environment)) return host;
    return host.to(environment);
}

inline Tensor loads(std::vector<std::byte> const& image, Environment environment = Host{}) { return loads(image.data(), image.size(), environment); }

inline void save(Tensor const& tensor, std::string const& path) {
    const std::vector<std::byte> image = dumps(tensor);
    std::FILE* file = std::fopen(path.c_str(), "wb");
    if (!file) throw Exception("save: cannot open " + path);
    const size_t written = std::fwrite(image.data(), 1, image.size(), file);
    const bool closed = std::fclose(file) == 0;
    if (written != image.size() || !closed) throw Exception("save: cannot write " + path);
}

inline Tensor load(std::string const& path, Environment environment = Host{}) {
    std::FILE* file = std::fopen(path.c_str(), "rb");
    if (!file) throw Exception("load: cannot open " + path);
    std::vector<std::byte> image;
    std::byte block[1 << 16];
    for (size_t got; (got = std::fread(block, 1, sizeof block, file)) > 0;) image.insert(image.end(), block, block + got);
    std::fclose(file);
    return loads(image, environment);
}

}  // namespace tannic::hip
