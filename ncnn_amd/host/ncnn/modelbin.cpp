#include "modelbin.h"

#include <stdint.h>
#include <string.h>

#include <vector>

#include "datareader.h"

namespace ncnn {

ModelBin::~ModelBin() {}

Mat ModelBin::load(int w, int h, int type) const
{
    Mat flat = load(w * h, type);
    return flat.empty() ? flat : flat.reshape(w, h);
}

Mat ModelBin::load(int w, int h, int c, int type) const
{
    Mat flat = load(w * h * c, type);
    return flat.empty() ? flat : flat.reshape(w, h, c);
}

Mat ModelBin::load(int w, int h, int d, int c, int type) const
{
    Mat flat = load(w * h * d * c, type);
    if (flat.empty()) return flat;
    Mat m;
    m.create(w, h, d, c, flat.elemsize);
    if (m.empty()) return m;
    const size_t plane = (size_t)w * h * d;
    for (int q = 0; q < c; q++)
        memcpy((unsigned char*)m.data + m.cstep * q * m.elemsize, (const unsigned char*)flat.data + plane * q * flat.elemsize, plane * flat.elemsize);
    return m;
}

ModelBinFromDataReader::ModelBinFromDataReader(const DataReader& _dr) : dr(_dr) {}

// payload of `bytes` bytes as a Mat of `w` elements: referenced in place when the reader can,
// copied otherwise
static Mat take_payload(const DataReader& dr, int w, size_t elemsize, size_t bytes, const char* what)
{
    const void* ref = 0;
    if (dr.reference(bytes, &ref) == bytes) return Mat(w, (void*)ref, elemsize);
    std::vector<unsigned char> tmp(bytes);
    const size_t got = bytes ? dr.read(tmp.data(), bytes) : 0;
    if (got != bytes)
    {
        NCNN_LOGE("ModelBin read %s failed %zd", what, got);
        return Mat();
    }
    Mat m(w, elemsize);
    if (!m.empty()) memcpy(m.data, tmp.data(), (size_t)w * elemsize);
    return m;
}

Mat ModelBinFromDataReader::load(int w, int type) const
{
    if (type == 1) return take_payload(dr, w, 4u, (size_t)w * 4, "weight_data");
    if (type != 0)
    {
        NCNN_LOGE("ModelBin load type %d not implemented", type);
        return Mat();
    }

    unsigned char tagbytes[4];
    const size_t got = dr.read(tagbytes, 4);
    if (got != 4)
    {
        NCNN_LOGE("ModelBin read flag_struct failed %zd", got);
        return Mat();
    }
    const uint32_t tag = (uint32_t)tagbytes[0] | ((uint32_t)tagbytes[1] << 8) | ((uint32_t)tagbytes[2] << 16) | ((uint32_t)tagbytes[3] << 24);

    if (tag == 0x01306B47u)
    {
        const size_t bytes = alignSize((size_t)w * 2, 4);
        Mat half = take_payload(dr, (int)(bytes / 2), 2u, bytes, "float16_weights");
        if (half.empty()) return half;
        return Mat::from_float16((const unsigned short*)half.data, w);
    }
    if (tag == 0x000D4B38u) return take_payload(dr, w, 1u, alignSize((size_t)w, 4), "int8_weights");
    if (tag == 0x0002C056u) return take_payload(dr, w, 4u, (size_t)w * 4, "weight_data");

    // the reference tests the byte SUM of the tag for "table-coded", then byte 0 for "raw"
    const unsigned byte_sum = (unsigned)tagbytes[0] + tagbytes[1] + tagbytes[2] + tagbytes[3];
    if (byte_sum != 0)
    {
        float table[256];
        if (dr.read(table, sizeof(table)) != sizeof(table))
        {
            NCNN_LOGE("ModelBin read quantization_value failed");
            return Mat();
        }
        const size_t bytes = alignSize((size_t)w, 4);
        std::vector<unsigned char> index(bytes);
        if (dr.read(index.data(), bytes) != bytes)
        {
            NCNN_LOGE("ModelBin read index_array failed");
            return Mat();
        }
        Mat m(w);
        if (m.empty()) return m;
        float* p = m;
        for (int i = 0; i < w; i++) p[i] = table[index[i]];
        return m;
    }
    return take_payload(dr, w, 4u, (size_t)w * 4, "weight_data");
}

ModelBinFromMatArray::ModelBinFromMatArray(const Mat* weights) : next(weights) {}

Mat ModelBinFromMatArray::load(int /*w*/, int /*type*/) const
{
    if (!next) return Mat();
    Mat m = *next;
    next++;
    return m;
}

} // namespace ncnn
