// Per-layer key=value table parsed from one .param line (src/paramdict.h:17-63).
// At most 32 ids.  A slot remembers how it was written: 2 int, 3 float, 4 array (set from code),
// 5 int array, 6 float array, 7 string.  get(id, def) returns def only for an unset slot and
// otherwise the stored value of the REQUESTED C type without conversion: an int literal read
// back as float yields the int's bit pattern, exactly like the reference (its storage is a
// union), which is why .param writers must spell floats with '.' or 'e'.
#ifndef NCNN_PARAMDICT_H
#define NCNN_PARAMDICT_H

#include <string>

#include "mat.h"

#define NCNN_MAX_PARAM_COUNT 32

namespace ncnn {

class DataReader;
class Net;
class NCNN_EXPORT ParamDict
{
public:
    ParamDict();
    ParamDict(const ParamDict&);
    ParamDict& operator=(const ParamDict&);
    virtual ~ParamDict();

    int type(int id) const;
    int get(int id, int def) const;
    float get(int id, float def) const;
    Mat get(int id, const Mat& def) const;
    std::string get(int id, const std::string& def) const;

    void set(int id, int i);
    void set(int id, float f);
    void set(int id, const Mat& v);
    void set(int id, const std::string& s);

    // exposed for the net loader and for tests
    void clear();
    int load_param(const DataReader& dr);
    int load_param_bin(const DataReader& dr);

private:
    struct Slot
    {
        int type;
        union
        {
            int i;
            float f;
        };
        Mat v;
        std::string s;
    };
    Slot* const slots;
};

} // namespace ncnn

#endif // NCNN_PARAMDICT_H
