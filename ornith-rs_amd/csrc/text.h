// Host-side text helpers shared by the tokenizer and the chat template: UTF-8 in and out,
// Unicode classes from the generated tables, NFC.
#pragma once

#include <stdint.h>

#include <string>
#include <vector>

namespace orn_text {

// Strict UTF-8 -> code points. False when the bytes are not well-formed UTF-8 (the reference
// takes Rust `&str`, which cannot hold anything else).
bool utf8_decode(const char* s, size_t n, std::vector<uint32_t>* out);
void utf8_append(std::string& s, uint32_t cp);
// Bytes -> text the way Rust's String::from_utf8_lossy and Python's
// bytes.decode("utf-8", "replace") do it: every maximal ill-formed subpart becomes one U+FFFD.
std::string utf8_lossy(const std::string& bytes);

bool is_letter(uint32_t c);       // \p{L}
bool is_mark(uint32_t c);         // \p{M}
bool is_number(uint32_t c);       // \p{N}
bool is_space(uint32_t c);        // \s as oniguruma reads it: the White_Space property
bool is_py_space(uint32_t c);     // Python's str.isspace()
int combining_class(uint32_t c);  // canonical combining class

// NFC (UAX #15) of a code point sequence.
std::vector<uint32_t> nfc(const std::vector<uint32_t>& s);

}  // namespace orn_text
