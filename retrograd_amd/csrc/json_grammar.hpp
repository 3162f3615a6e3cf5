// The grammar behind retro_grammar_json_object (reference retro_lora_train.h:1397-1400: "the built-in any-JSON
// grammar"; the reference embeds llama.cpp's grammars/json.gbnf, absent from its checkout): one JSON object as
// RFC 8259 defines it, white space allowed after every token, written for this library.
#pragma once

namespace retro {

static const char * const kJsonObjectGbnf = R"GBNF(root   ::= object
value  ::= object | array | string | number | ("true" | "false" | "null") ws
object ::= "{" ws ( string ":" ws value ("," ws string ":" ws value)* )? "}" ws
array  ::= "[" ws ( value ("," ws value)* )? "]" ws
string ::= "\"" ( [^"\\\x00-\x1F] | "\\" ( ["\\/bfnrt] | "u" [0-9a-fA-F]{4} ) )* "\"" ws
number ::= "-"? ( "0" | [1-9] [0-9]* ) ( "." [0-9]+ )? ( [eE] [-+]? [0-9]+ )? ws
ws     ::= [ \t\n\r]*
)GBNF";

}  // namespace retro
