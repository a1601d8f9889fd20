#include "paramdict.h"

#include <ctype.h>
#include <stdio.h>
#include <string.h>

#include <vector>

#include "datareader.h"

namespace ncnn {

ParamDict::ParamDict() : slots(new Slot[NCNN_MAX_PARAM_COUNT])
{
    clear();
}

ParamDict::ParamDict(const ParamDict& rhs) : slots(new Slot[NCNN_MAX_PARAM_COUNT])
{
    *this = rhs;
}

ParamDict& ParamDict::operator=(const ParamDict& rhs)
{
    if (this == &rhs) return *this;
    for (int k = 0; k < NCNN_MAX_PARAM_COUNT; k++)
    {
        slots[k].type = rhs.slots[k].type;
        slots[k].i = rhs.slots[k].i;
        slots[k].v = rhs.slots[k].v;
        slots[k].s = rhs.slots[k].s;
    }
    return *this;
}

ParamDict::~ParamDict()
{
    delete[] slots;
}

void ParamDict::clear()
{
    for (int k = 0; k < NCNN_MAX_PARAM_COUNT; k++)
    {
        slots[k].type = 0;
        slots[k].i = 0;
        slots[k].v = Mat();
        slots[k].s.clear();
    }
}

int ParamDict::type(int id) const
{
    return slots[id].type;
}
int ParamDict::get(int id, int def) const
{
    return slots[id].type ? slots[id].i : def;
}
float ParamDict::get(int id, float def) const
{
    return slots[id].type ? slots[id].f : def;
}
Mat ParamDict::get(int id, const Mat& def) const
{
    return slots[id].type ? slots[id].v : def;
}
std::string ParamDict::get(int id, const std::string& def) const
{
    return slots[id].type ? slots[id].s : def;
}

void ParamDict::set(int id, int i)
{
    slots[id].type = 2;
    slots[id].i = i;
}
void ParamDict::set(int id, float f)
{
    slots[id].type = 3;
    slots[id].f = f;
}
void ParamDict::set(int id, const Mat& v)
{
    slots[id].type = 4;
    slots[id].v = v;
}
void ParamDict::set(int id, const std::string& s)
{
    slots[id].type = 7;
    slots[id].s = s;
}

// A token is a float iff it contains '.' or an exponent letter (src/paramdict.cpp:163-176).
static bool token_is_float(const char* t)
{
    for (; *t; t++)
        if (*t == '.' || *t == 'e' || *t == 'E') return true;
    return false;
}

// Decimal text -> float the way the reference does it (src/paramdict.cpp:183-258): integer
// digits and fraction digits are gathered as 32-bit unsigned integers, combined in double as
// int + frac/10^digits, scaled by 10^exp through repeated multiplication (1e8 steps, then 10),
// and only then rounded to float.  Reproducing that recipe (rather than calling strtof) keeps
// every parsed parameter bit-identical to what ncnn would hold.
static float token_to_float(const char* t)
{
    bool negative = false;
    if (*t == '+' || *t == '-') negative = *t++ == '-';

    unsigned whole = 0;
    for (; isdigit((unsigned char)*t); t++) whole = whole * 10u + (unsigned)(*t - '0');
    double value = (double)whole;

    if (*t == '.')
    {
        t++;
        unsigned frac = 0, denom = 1;
        for (; isdigit((unsigned char)*t); t++)
        {
            frac = frac * 10u + (unsigned)(*t - '0');
            denom *= 10u;
        }
        value += frac / (double)denom;
    }

    if (*t == 'e' || *t == 'E')
    {
        t++;
        bool exp_negative = false;
        if (*t == '+' || *t == '-') exp_negative = *t++ == '-';
        unsigned e = 0;
        for (; isdigit((unsigned char)*t); t++) e = e * 10u + (unsigned)(*t - '0');
        double scale = 1.0;
        for (; e >= 8; e -= 8) scale *= 1e8;
        for (; e > 0; e--) scale *= 10.0;
        value = exp_negative ? value / scale : value * scale;
    }
    return negative ? (float)-value : (float)value;
}

static bool token_to_int(const char* t, int* out)
{
    return sscanf(t, "%d", out) == 1;
}

int ParamDict::load_param(const DataReader& dr)
{
    clear();

    // forms:  7=3   1=1.25   10=0.0,6.0   -23310=2,0.0,6.0 (legacy counted array)   5="text"
    int id = 0;
    while (dr.scan("%d=", &id) == 1)
    {
        const bool counted_array = id <= -23300;
        if (counted_array) id = -id - 23300;
        if (id < 0 || id >= NCNN_MAX_PARAM_COUNT)
        {
            NCNN_LOGE("id < NCNN_MAX_PARAM_COUNT failed (id=%d, NCNN_MAX_PARAM_COUNT=%d)", id, NCNN_MAX_PARAM_COUNT);
            return -1;
        }
        Slot& slot = slots[id];
        char tok[16];

        if (counted_array)
        {
            int len = 0;
            if (dr.scan("%d", &len) != 1 || len < 0 || len > (1 << 24))
            {
                NCNN_LOGE("ParamDict read array length failed");
                return -1;
            }
            slot.v.create(len);
            bool any_float = false;
            for (int j = 0; j < len; j++)
            {
                if (dr.scan(",%15[^,\n ]", tok) != 1)
                {
                    NCNN_LOGE("ParamDict read array element failed");
                    return -1;
                }
                any_float = token_is_float(tok);
                if (any_float)
                    ((float*)slot.v.data)[j] = token_to_float(tok);
                else if (!token_to_int(tok, (int*)slot.v.data + j))
                {
                    NCNN_LOGE("ParamDict parse array element failed");
                    return -1;
                }
                slot.type = any_float ? 6 : 5;
            }
            continue;
        }

        if (dr.scan("%15[^,\n ]", tok) != 1)
        {
            NCNN_LOGE("ParamDict read value failed");
            return -1;
        }

        if (isalpha((unsigned char)tok[0]) || tok[0] == '"')
        {
            // string value, possibly longer than the first token or quoted
            std::string text = tok[0] == '"' ? tok + 1 : tok;
            char more[256];
            const bool quoted_open = tok[0] == '"' && tok[strlen(tok) - 1] != '"';
            int got = 0;
            if (tok[0] != '"')
                got = dr.scan("%255[^\n ]", more);
            else if (quoted_open)
                got = dr.scan("%255[^\"\n]\"", more);
            if (got == 1) text += more;
            if (text.size() > 255)
            {
                NCNN_LOGE("string too long (id=%d)", id);
                return -1;
            }
            if (!text.empty() && text[text.size() - 1] == '"') text.resize(text.size() - 1);
            slot.s = text;
            slot.type = 7;
            continue;
        }

        const bool is_float = token_is_float(tok);
        char comma[4];
        if (dr.scan("%1[,]", comma) == 1)
        {
            // comma list; the first token decides int vs float for the whole array
            std::vector<float> fv;
            std::vector<int> iv;
            for (;;)
            {
                if (is_float)
                    fv.push_back(token_to_float(tok));
                else
                {
                    int v = 0;
                    if (!token_to_int(tok, &v))
                    {
                        NCNN_LOGE("ParamDict parse value failed");
                        return -1;
                    }
                    iv.push_back(v);
                }
                if (fv.size() + iv.size() > 1 && dr.scan("%1[,]", comma) != 1) break;
                if (dr.scan("%15[^,\n ]", tok) != 1) break;
            }
            const size_t count = is_float ? fv.size() : iv.size();
            slot.v.create((int)count);
            memcpy(slot.v.data, is_float ? (const void*)fv.data() : (const void*)iv.data(), count * 4);
            slot.type = is_float ? 6 : 5;
        }
        else
        {
            if (is_float)
                slot.f = token_to_float(tok);
            else if (!token_to_int(tok, &slot.i))
            {
                NCNN_LOGE("ParamDict parse value failed");
                return -1;
            }
            slot.type = is_float ? 3 : 2;
        }
    }
    return 0;
}

// The binary form of a layer's parameters (src/paramdict.cpp:491-637): little-endian 32-bit words, `id value` pairs up to
// the end mark -233.  An id <= -23300 announces an array (id = -id - 23300; a length word, then that many 32-bit values),
// an id <= -23400 a string (id = -id - 23400; a length word of at most 255, then the bytes padded to whole words).  The
// file does not say whether a value is an int or a float: a scalar gets type 1 and an array type 4, and the getters hand
// out the stored bits either way.
int ParamDict::load_param_bin(const DataReader& dr)
{
    clear();
    int id = 0;
    if (dr.read(&id, 4) != 4)
    {
        NCNN_LOGE("ParamDict read id failed");
        return -1;
    }
    while (id != -233)
    {
        const bool is_string = id <= -23400, is_array = id <= -23300;
        if (is_string)
            id = -id - 23400;
        else if (is_array)
            id = -id - 23300;
        if (id < 0 || id >= NCNN_MAX_PARAM_COUNT)
        {
            NCNN_LOGE("id < NCNN_MAX_PARAM_COUNT failed (id=%d, NCNN_MAX_PARAM_COUNT=%d)", id, NCNN_MAX_PARAM_COUNT);
            return -1;
        }
        Slot& slot = slots[id];
        if (is_string || is_array)
        {
            int len = 0;
            if (dr.read(&len, 4) != 4 || len < 0 || len > (is_string ? 255 : (1 << 24)))
            {
                NCNN_LOGE("ParamDict read %s length failed (id=%d)", is_string ? "string" : "array", id);
                return -1;
            }
            if (is_string)
            {
                char text[260];
                const size_t padded = ((size_t)len + 3) / 4 * 4;
                if (dr.read(text, padded) != padded)
                {
                    NCNN_LOGE("ParamDict read string failed");
                    return -1;
                }
                text[padded] = 0;
                slot.s = text; // up to the first zero byte, as the reference assigns it
                slot.type = 7;
            }
            else
            {
                slot.v.create(len);
                if (len > 0 && (slot.v.empty() || dr.read(slot.v.data, (size_t)len * 4) != (size_t)len * 4))
                {
                    NCNN_LOGE("ParamDict read array element failed");
                    return -1;
                }
                slot.type = 4;
            }
        }
        else
        {
            if (dr.read(&slot.f, 4) != 4)
            {
                NCNN_LOGE("ParamDict read value failed");
                return -1;
            }
            slot.type = 1;
        }
        if (dr.read(&id, 4) != 4)
        {
            NCNN_LOGE("ParamDict read EOP failed");
            return -1;
        }
    }
    return 0;
}

} // namespace ncnn
