// One edge of the graph (src/blob.h): its name, the layer that writes it, the layer that reads it.
#ifndef NCNN_BLOB_H
#define NCNN_BLOB_H

#include <string>

#include "mat.h"

namespace ncnn {

class NCNN_EXPORT Blob
{
public:
    Blob() : producer(-1), consumer(-1) {}
    std::string name;
    int producer;
    int consumer;
    Mat shape;
};

} // namespace ncnn

#endif // NCNN_BLOB_H
