// Prints the GBNF text the library's converter makes of a JSON schema (retrograd_amd/csrc/json_schema.hpp), or
// "error: ..."; driven by tests/test_grammar.py. CPU only.
//   schema_unit <schema file>
#include <cstdio>
#include <fstream>
#include <iterator>

#include "../../retrograd_amd/csrc/grammar.hpp"
#include "../../retrograd_amd/csrc/json_schema.hpp"

int main(int argc, char ** argv) {
    if (argc != 2) return 2;
    std::ifstream in(argv[1], std::ios::binary);
    const std::string schema((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    try {
        const std::string gbnf = retro::SchemaToGbnf::convert(schema);
        retro::Grammar check(gbnf);          // what the converter writes must parse
        std::fputs(gbnf.c_str(), stdout);
    } catch (const std::exception & e) {
        std::printf("error: %s\n", e.what());
        return 1;
    }
    return 0;
}
