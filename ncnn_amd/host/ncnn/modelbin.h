// Reader of the .bin weight stream (interface of src/modelbin.h).
// load(w, type): type 0 = tagged weight blob (4-byte tag, payload padded to 4 bytes):
//     0x01306B47 fp16 (expanded to fp32)   0x000D4B38 int8 (kept, elemsize 1)
//     0x0002C056 fp32 raw                  0 fp32 raw
//     any other tag: 256-entry fp32 table followed by one index byte per weight
//   type 1 = raw fp32 without tag (bias and scale tables).
#ifndef NCNN_MODELBIN_H
#define NCNN_MODELBIN_H

#include "mat.h"

namespace ncnn {

class DataReader;
class NCNN_EXPORT ModelBin
{
public:
    virtual ~ModelBin();
    virtual Mat load(int w, int type) const = 0;
    virtual Mat load(int w, int h, int type) const;
    virtual Mat load(int w, int h, int c, int type) const;
    virtual Mat load(int w, int h, int d, int c, int type) const;
};

class NCNN_EXPORT ModelBinFromDataReader : public ModelBin
{
public:
    explicit ModelBinFromDataReader(const DataReader& dr);
    virtual Mat load(int w, int type) const;

private:
    const DataReader& dr;
};

// weights handed over as an array of Mats, consumed in order (used by layer unit tests)
class NCNN_EXPORT ModelBinFromMatArray : public ModelBin
{
public:
    explicit ModelBinFromMatArray(const Mat* weights);
    virtual Mat load(int w, int type) const;

private:
    mutable const Mat* next;
};

} // namespace ncnn

#endif // NCNN_MODELBIN_H
