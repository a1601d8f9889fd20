#include "datareader.h"

#include <string.h>

#include <string>

namespace ncnn {

DataReader::~DataReader() {}
int DataReader::scan(const char*, void*) const
{
    return 0;
}
size_t DataReader::read(void*, size_t) const
{
    return 0;
}
size_t DataReader::reference(size_t, const void**) const
{
    return 0;
}

DataReaderFromStdio::DataReaderFromStdio(FILE* _fp) : fp(_fp) {}
int DataReaderFromStdio::scan(const char* format, void* p) const
{
    return fscanf(fp, format, p);
}
size_t DataReaderFromStdio::read(void* buf, size_t size) const
{
    return fread(buf, 1, size, fp);
}

DataReaderFromMemory::DataReaderFromMemory(const unsigned char*& _mem) : mem(_mem) {}
int DataReaderFromMemory::scan(const char* format, void* p) const
{
    // %n reports how much text the conversion consumed, so the cursor can follow
    std::string fmt(format);
    fmt += "%n";
    int consumed = 0;
    const int got = sscanf((const char*)mem, fmt.c_str(), p, &consumed);
    mem += consumed;
    return consumed > 0 ? got : 0;
}
size_t DataReaderFromMemory::read(void* buf, size_t size) const
{
    memcpy(buf, mem, size);
    mem += size;
    return size;
}
size_t DataReaderFromMemory::reference(size_t size, const void** buf) const
{
    *buf = mem;
    mem += size;
    return size;
}

} // namespace ncnn
