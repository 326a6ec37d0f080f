// tosa_mi355_run: command-line runner with the contract of the reference's tosa_reference_model for the
// accelerated path (reference_model/src/main.cpp:55-260): reads a test descriptor (desc.json), the TOSA
// flatbuffer and the .npy inputs it names, evaluates the graph on the GPU, writes the .npy outputs and exits
// with the GraphStatus (0 valid, 1 unpredictable, 2 error), which is what the reference's Python runner
// interprets (verif/runner/tosa_refmodel_sut_run.py:12-18,59-68).
//
//   tosa_mi355_run --test_desc=<dir>/desc.json [--ofm_file=<name>] [--flatbuffer_dir=<dir>] [--no_fusion]
//                  [--precise_mode=1] [--tosa_level=NONE|EIGHTK]
//
// --precise_mode=1 (reference_model/src/command_line_utils.h:65): floating-point CONV2D / DEPTHWISE_CONV2D /
// MATMUL results are computed and written in fp64; when the descriptor says
// test_requirements.bounds_file_required, the graph is evaluated a second time in bounds mode and those results
// go to "bounds_" + ofm_file (reference_model/src/main.cpp:109-121, :246-251, :404-407).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "tosa_host.h"

using namespace tmi_host;

namespace
{

// The descriptor only holds strings, booleans and arrays of strings: a scanner for those is enough.
struct Desc
{
    std::string tosa_file;
    std::vector<std::string> ifm_name, ifm_file, ofm_name, ofm_file;
    bool bounds_file_required = false;    // test_requirements.bounds_file_required
};

bool parse_string(const std::string& s, size_t& i, std::string& out)
{
    if (s[i] != '"')
        return false;
    out.clear();
    for (i++; i < s.size() && s[i] != '"'; i++)
    {
        if (s[i] == '\\' && i + 1 < s.size())
            i++;
        out += s[i];
    }
    if (i >= s.size())
        return false;
    i++;
    return true;
}

void skip_ws(const std::string& s, size_t& i)
{
    while (i < s.size() && (s[i] == ' ' || s[i] == '\n' || s[i] == '\t' || s[i] == '\r' || s[i] == ',' || s[i] == ':'))
        i++;
}

bool parse_desc(const std::string& text, Desc& d)
{
    size_t i = 0;
    while (i < text.size())
    {
        skip_ws(text, i);
        if (i >= text.size())
            break;
        if (text[i] == '{' || text[i] == '}')
        {
            i++;
            continue;
        }
        std::string key;
        if (!parse_string(text, i, key))
        {
            i++;
            continue;
        }
        skip_ws(text, i);
        std::vector<std::string> values;
        if (i < text.size() && text[i] == '[')
        {
            for (i++; i < text.size() && text[i] != ']';)
            {
                skip_ws(text, i);
                std::string v;
                if (i < text.size() && text[i] == '"')
                {
                    if (!parse_string(text, i, v))
                        return false;
                    values.push_back(v);
                }
                else if (i < text.size() && text[i] != ']')
                    i++;
            }
            i++;
        }
        else if (i < text.size() && text[i] == '"')
        {
            std::string v;
            if (!parse_string(text, i, v))
                return false;
            values.push_back(v);
        }
        else if (i < text.size() && text[i] == '{')
            continue;    // a nested object: its keys are read like top-level ones
        else
        {
            const size_t v0 = i;
            while (i < text.size() && text[i] != ',' && text[i] != '}')
                i++;
            if (key == "bounds_file_required")
                d.bounds_file_required = text.compare(v0, 4, "true") == 0;
        }
        if (key == "tosa_file" && !values.empty())
            d.tosa_file = values[0];
        else if (key == "ifm_name")
            d.ifm_name = values;
        else if (key == "ifm_file")
            d.ifm_file = values;
        else if (key == "ofm_name")
            d.ofm_name = values;
        else if (key == "ofm_file")
            d.ofm_file = values;
    }
    return !d.tosa_file.empty();
}

std::string dir_of(const std::string& p)
{
    const size_t k = p.find_last_of('/');
    return k == std::string::npos ? "." : p.substr(0, k);
}

int fail(const char* what, const std::string& msg)
{
    fprintf(stderr, "tosa_mi355_run: %s: %s\n", what, msg.c_str());
    return (int)GraphStatus::TOSA_ERROR;
}

}    // namespace

int main(int argc, char** argv)
{
    std::string test_desc, ofm_override, fb_dir;
    bool fusion = true, precise = false;
    tmi_level_t level = { 0, 0, 0, 0, 0 };
    for (int a = 1; a < argc; a++)
    {
        const std::string s = argv[a];
        auto val            = [&](const char* k) -> const char* {
            const size_t n = strlen(k);
            return s.compare(0, n, k) == 0 ? s.c_str() + n : nullptr;
        };
        if (const char* v = val("--test_desc="))
            test_desc = v;
        else if (const char* v = val("--ofm_file="))
            ofm_override = v;
        else if (const char* v = val("--flatbuffer_dir="))
            fb_dir = v;
        else if (s == "--no_fusion")
            fusion = false;
        else if (const char* v = val("--precise_mode="))
            precise = atoi(v) != 0;
        else if (const char* v = val("--tosa_level="))
        {
            // command_line_utils.h:62, main.cpp: NONE or EIGHTK (func_config.h:65)
            if (std::string(v) == "EIGHTK")
                level = tmi_level_t{ 6, 8192, 8192, 256, 64 };
            else if (std::string(v) == "NONE")
                level = tmi_level_t{ 0, 0, 0, 0, 0 };
            else
                return fail("unknown TOSA level", v);
        }
        else
            return fail("unknown argument", s);
    }
    if (test_desc.empty())
        return fail("usage", "--test_desc=<desc.json> is required");
    std::ifstream f(test_desc);
    if (!f)
        return fail("cannot open", test_desc);
    std::stringstream ss;
    ss << f.rdbuf();
    Desc desc;
    if (!parse_desc(ss.str(), desc))
        return fail("malformed test descriptor", test_desc);
    if (fb_dir.empty())
        fb_dir = dir_of(test_desc);
    if (desc.ifm_name.size() != desc.ifm_file.size() || desc.ofm_name.size() != desc.ofm_file.size())
        return fail("descriptor", "ifm/ofm name and file lists differ in length");

    BasicBlock block;
    std::string err;
    if (!load_tosa_file(fb_dir + "/" + desc.tosa_file, block, err))
        return fail("graph", err);

    // at most two runs; the second one only in precise mode, for the bounds results (reference: main.cpp:123-254)
    GraphStatus st = GraphStatus::TOSA_VALID;
    int kernels = 0, folded = 0;
    std::string message;
    for (int run = 0; run < (precise && desc.bounds_file_required ? 2 : 1); run++)
    {
        ModelRunner runner(0);
        if (!fusion)
            runner.disableFusion();
        runner.setPreciseMode(precise, run == 1, precise && desc.bounds_file_required);
        runner.setLevel(level);
        st = runner.initialize(block);
        if (st != GraphStatus::TOSA_VALID)
        {
            fprintf(stderr, "Graph result: %s (%s)\n", st == GraphStatus::TOSA_UNPREDICTABLE ? "UNPREDICTABLE" : "ERROR",
                    runner.traverser() ? runner.traverser()->last_message.c_str() : "");
            return (int)st;
        }
        for (size_t i = 0; i < desc.ifm_name.size(); i++)
        {
            NpyArray arr;
            if (!read_npy(fb_dir + "/" + desc.ifm_file[i], arr, err))
                return fail("input", err);
            Tensor* t = runner.traverser()->findTensorByName(desc.ifm_name[i]);
            if (!t)
                return fail("input", "no tensor named " + desc.ifm_name[i]);
            if (arr.descr != npy_descr_for(t->getDtype()) && !(arr.descr == "<i1" && t->getDtype() == DType_INT8))
                return fail("input", desc.ifm_file[i] + ": descr " + arr.descr + " does not match the tensor type");
            if (arr.shape != t->getShape() || arr.data.size() < t->bytes())
                return fail("input", desc.ifm_file[i] + ": shape does not match tensor " + desc.ifm_name[i]);
            if (runner.setInput(desc.ifm_name[i], arr.data.data(), t->bytes()))
                return fail("input", "setInput failed for " + desc.ifm_name[i]);
        }
        st = runner.run();
        SubgraphTraverser* sgt = runner.traverser();
        if (st == GraphStatus::TOSA_ERROR)
        {
            fprintf(stderr, "Graph result: ERROR (%s)\n", sgt->last_message.c_str());
            return (int)st;
        }
        for (size_t i = 0; i < desc.ofm_name.size(); i++)
        {
            Tensor* t = sgt->findTensorByName(desc.ofm_name[i]);
            if (!t || !t->host_valid)
                return fail("output", "no result for " + desc.ofm_name[i]);
            std::string name = (i == 0 && !ofm_override.empty()) ? ofm_override : desc.ofm_file[i];
            if (run == 1)
            {
                const size_t k = name.find_last_of('/');
                name.insert(k == std::string::npos ? 0 : k + 1, "bounds_");
            }
            if (name.empty() || name[0] != '/')
                name = fb_dir + "/" + name;
            if (!write_npy(name, t->precise ? "<f8" : npy_descr_for(t->getDtype()), t->getShape(), t->host.data(),
                           t->bytes(), err))
                return fail("output", err);
        }
        kernels += sgt->kernels_launched, folded += sgt->nodes_folded;
        message = sgt->last_message;
        if (st != GraphStatus::TOSA_VALID)
            break;    // the bounds run only follows a valid first run
    }
    fprintf(stderr, "Graph result: %s (kernels launched: %d, nodes folded into a producer: %d)\n",
            st == GraphStatus::TOSA_VALID ? "VALID" : "UNPREDICTABLE", kernels, folded);
    if (st != GraphStatus::TOSA_VALID)
        fprintf(stderr, "%s\n", message.c_str());
    return (int)st;
}
