// reserialize: read a serialized model and write it back (nGraph's tool of the same name,
// src/tools/reserialize/reserialize.cpp:34-126; its constant-to-broadcast option is not offered).
// An indent of 0 (the default, as in nGraph) writes the compact form.  An input named *.onnx or
// *.prototxt is read as an ONNX model instead (binary or text), which makes this the converter from
// ONNX to the serialized form nbench takes.
#include <chrono>
#include <fstream>
#include <iostream>
#include <string>

#include "ngraph/frontend/onnx_import/onnx.hpp"
#include "ngraph/serializer.hpp"

using namespace std;

static void help()
{
    cout << R"###(
DESCRIPTION
    Reserialize a serialized model

SYNOPSIS
        reserialize [-i|--input <input file>] [-o|--output <output file>] [--indent <n>]

OPTIONS
        -i or --input  input serialized model (or an ONNX model: *.onnx, *.prototxt)
        -o or --output output serialized model
        --indent       pretty-print with this many blanks per level
)###";
}

int main(int argc, char** argv)
{
    string input, output;
    size_t indent = 0;
    for (int i = 1; i < argc; i++)
    {
        string arg = argv[i];
        if ((arg == "-o" || arg == "--output") && i + 1 < argc)
            output = argv[++i];
        else if ((arg == "-i" || arg == "--input") && i + 1 < argc)
            input = argv[++i];
        else if (arg == "--indent" && i + 1 < argc)
            indent = static_cast<size_t>(stoul(argv[++i]));
        else if (arg == "-h" || arg == "--help")
        {
            help();
            return 0;
        }
        else
        {
            cout << "Unknown option: " << arg << endl;
            help();
            return 1;
        }
    }
    if (input.empty())
    {
        cout << "input file missing\n";
        help();
        return 1;
    }
    if (output.empty())
    {
        cout << "output file missing\n";
        help();
        return 1;
    }
    ifstream f(input);
    if (!f)
    {
        cout << "failed to open '" << input << "' for input\n";
        return 2;
    }
    try
    {
        auto t0 = chrono::steady_clock::now();
        auto ends_with = [&](const string& tail) { return input.size() >= tail.size() && input.compare(input.size() - tail.size(), tail.size(), tail) == 0; };
        const bool onnx = ends_with(".onnx") || ends_with(".prototxt");
        shared_ptr<ngraph::Function> function = onnx ? ngraph::onnx_import::import_onnx_model(f) : ngraph::deserialize(f);
        auto t1 = chrono::steady_clock::now();
        cout << (onnx ? "onnx import took " : "deserialize took ") << chrono::duration<double, milli>(t1 - t0).count() << "ms\n";
        ngraph::serialize(output, function, indent);
        auto t2 = chrono::steady_clock::now();
        cout << "serialize took   " << chrono::duration<double, milli>(t2 - t1).count() << "ms\n";
    }
    catch (const exception& e)
    {
        cout << e.what() << endl;
        return 3;
    }
    return 0;
}
