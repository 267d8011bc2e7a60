// NCHW tensor of the layer graph: host-side shape, DEVICE-side data.  Interface
// of feather::Blob (utility/blob.h:24-120 of the reference); the data pointer
// addresses memory of the device arena, obtained through a RangeAllocator, and
// CopyData()/CopyToHost() cross the host/device boundary.
#pragma once

#include <assert.h>
#include <stdio.h>

#include <string>

#include "device.h"
#include "range_allocator.h"

namespace feather {

template <class Dtype>
class Blob {
   public:
    Blob() : _data(NULL), _num(0), _channels(0), _height(0), _width(0), _alloc(NULL), _owned(false) {}

    explicit Blob(const size_t num, const size_t channels, const size_t height, const size_t width)
        : _data(NULL), _num(num), _channels(channels), _height(height), _width(width), _name(), _alloc(NULL),
          _owned(false) {}

    // Wraps device memory the caller owns.
    explicit Blob(Dtype *data, const size_t num, const size_t channels, const size_t height, const size_t width)
        : _data(data), _num(num), _channels(channels), _height(height), _width(width), _name(), _alloc(NULL),
          _owned(false) {}

    explicit Blob(Dtype *data, size_t num, size_t channels, size_t height, size_t width, std::string name)
        : _data(data), _num(num), _channels(channels), _height(height), _width(width), _name(name), _alloc(NULL),
          _owned(false) {}

    ~Blob() { Free(); }

    // Where Alloc() takes device memory from.
    void SetAllocator(fastconv::RangeAllocator *alloc) { _alloc = alloc; }

    void Free() {
        if (_owned && _data && _alloc) _alloc->Free(_data);
        _data = NULL;
        _owned = false;
    }
    void Alloc() {
        assert(_alloc != NULL);
        Free();
        const size_t bytes = data_size() * sizeof(Dtype);
        _data = bytes ? (Dtype *)_alloc->Allocate(bytes) : NULL;
        _owned = _data != NULL;
        if (bytes && !_data) fprintf(stderr, "Error: cannot allocate %zu bytes for blob %s\n", bytes, _name.c_str());
    }

    void ReshapeWithRealloc(const Blob<Dtype> *p_blob) {
        ReshapeWithRealloc((int)p_blob->num(), (int)p_blob->channels(), (int)p_blob->height(), (int)p_blob->width());
    }
    void ReshapeWithRealloc(int num, int channels, int height, int width) {
        const size_t elem_size = (size_t)num * channels * height * width;
        Realloc(elem_size);
        _num = num;
        _channels = channels;
        _height = height;
        _width = width;
    }
    // Grows the device buffer to hold elem_size elements (contents are not kept).
    void Realloc(size_t elem_size) {
        if (elem_size > data_size() || !_data) {
            assert(_alloc != NULL);
            Free();
            _data = (Dtype *)_alloc->Allocate(elem_size * sizeof(Dtype));
            _owned = _data != NULL;
        }
    }

    // host -> device
    void CopyData(const Dtype *data) {
        fastconv::Device &d = fastconv::Device::Get();
        d.Check(fc_upload(d.ctx(), _data, data, sizeof(Dtype) * data_size()), "Blob::CopyData");
    }
    // device -> host
    void CopyToHost(Dtype *data) const {
        fastconv::Device &d = fastconv::Device::Get();
        d.Check(fc_download(d.ctx(), data, _data, sizeof(Dtype) * data_size()), "Blob::CopyToHost");
    }
    void CopyShape(const Blob<Dtype> *p_blob) {
        this->_num = p_blob->num();
        this->_channels = p_blob->channels();
        this->_width = p_blob->width();
        this->_height = p_blob->height();
    }

    Dtype *data() const { return _data; }
    size_t data_size() const { return _num * _channels * _height * _width; }
    std::string name() { return _name; }
    size_t num() const { return _num; }
    size_t channels() const { return _channels; }
    size_t height() const { return _height; }
    size_t width() const { return _width; }
    void PrintBlobInfo() const {
        printf("----BlobInfo----\n");
        printf("Shape in nchw (%zu %zu %zu %zu)\n", _num, _channels, _height, _width);
        printf("----------------\n");
    }

   private:
    Dtype *_data;
    size_t _num;
    size_t _channels;
    size_t _height;
    size_t _width;
    std::string _name;
    fastconv::RangeAllocator *_alloc;
    bool _owned;
};

}  // namespace feather
