// Runs the host half of the model loader (fdx_model_check: JSON reader, base64 decoder, graph builder, load-time fusion,
// shape inference) over a list of files.  Built with -fsanitize=address,undefined together with the loader's source, so
// that a malformed file which makes the loader read or write out of bounds, overflow or misuse a pointer ends the
// program with a report instead of passing silently.  Usage: loader_sanitize <list-file>, one path per line; prints
// "<status> <path>" per file.
#include <cstdio>
#include <fstream>
#include <iterator>
#include <string>
#include <vector>

#include "../../include/fdx.h"

int main(int argc, char** argv)
{
    if (argc != 2)
        return 2;
    std::ifstream list(argv[1]);
    std::string path;
    int files = 0;
    while (std::getline(list, path)) {
        std::ifstream f(path, std::ios::binary);
        if (!f)
            return 3;
        const std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
        // a heap copy of exactly the file's length: reads past the end are then visible to the sanitizer
        std::vector<char> exact(text.begin(), text.end());
        const fdx_status st = fdx_model_check(exact.data(), exact.size(), 7);
        std::printf("%d %s\n", (int)st, path.c_str());
        ++files;
    }
    std::printf("loader_sanitize done: %d files\n", files);
    return 0;
}
