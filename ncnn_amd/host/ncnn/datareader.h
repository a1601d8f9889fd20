// Sources of .param text and .bin bytes (interface of src/datareader.h).
#ifndef NCNN_DATAREADER_H
#define NCNN_DATAREADER_H

#include <stddef.h>
#include <stdio.h>

#include "platform.h"

namespace ncnn {

class NCNN_EXPORT DataReader
{
public:
    virtual ~DataReader();
    // sscanf-style read of one item of the param text; returns the number of items read
    virtual int scan(const char* format, void* p) const;
    // returns bytes read
    virtual size_t read(void* buf, size_t size) const;
    // zero-copy: hand out a pointer into the model bytes; returns bytes referenced (0 = unsupported)
    virtual size_t reference(size_t size, const void** buf) const;
};

class NCNN_EXPORT DataReaderFromStdio : public DataReader
{
public:
    explicit DataReaderFromStdio(FILE* fp);
    virtual int scan(const char* format, void* p) const;
    virtual size_t read(void* buf, size_t size) const;

private:
    FILE* fp;
};

class NCNN_EXPORT DataReaderFromMemory : public DataReader
{
public:
    // mem is advanced as data is consumed
    explicit DataReaderFromMemory(const unsigned char*& mem);
    virtual int scan(const char* format, void* p) const;
    virtual size_t read(void* buf, size_t size) const;
    virtual size_t reference(size_t size, const void** buf) const;

private:
    const unsigned char*& mem;
};

} // namespace ncnn

#endif // NCNN_DATAREADER_H
