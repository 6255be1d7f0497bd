// Tokenizer of the reference (src/tokenizer/tokenizer.cu:21-155,200-343): a byte trie over the
// vocabulary of a Hugging Face tokenizer.json ("model"."vocab" and "added_tokens"), greedy longest
// match from the current byte, and a decode table id -> string.  Not BPE-merge exact, as in the
// reference.  The reference reads model_weights/modified_tokenizer.json (tokenizer.json with the byte
// markers for space and newline replaced, setup-tokenizer.py); load_tokenizer_from() takes the path and
// the table size instead.  Same structs, same names, same messages and exit(1) on failure; unlike the
// reference the decode table is zero-initialised, a missing "added_tokens" is reported as such, nodes are
// released by free_tokenizer(), a node's children are kept sorted by byte (binary search instead of a scan;
// the vocabulary is laid down from a sorted list in one pass), and tokenize() starts every token from a
// 256-entry table of the root's children.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <string>
#include <vector>

#include <sys/stat.h>

#include "common/fail.h"
#include "llama3_host.h"
#include "safetensor/json.h"

// Size of the decode table that the reference-named _build_decoder() checks ids against (its signature
// carries no size).  Per thread, set by the load that is running on that thread; loads on different
// threads do not see each other's value.
static thread_local int g_decode_size = 128256;

extern "C" {

// tokenizer.cu:231-245: size of a file in bytes, -1 (and a message through perror) when it cannot be examined
long _get_file_size(const char *filename) {
    struct stat st;
    if (stat(filename, &st) != 0) {
        perror("Failed to open file");
        return -1;
    }
    return (long)st.st_size;
}

// tokenizer.cu:200-229: the whole file as one NUL-terminated string that the caller frees.  One open: the size
// comes from the descriptor that is then read, so a file replaced between the two steps cannot overrun.
char *read_tokenizer_json(Llama3Tokenizer *tokenizer, const char *filename) {
    (void)tokenizer;
    FILE *in = fopen(filename, "rb");
    struct stat st;
    if (in == NULL || fstat(fileno(in), &st) != 0) { // the reference's two messages for a file it cannot size
        perror("Failed to open file");
        if (in) fclose(in);
        llama3_fail("Could not determine file size");
    }
    const size_t want = (size_t)st.st_size;
    char *text = (char *)malloc(want + 1);
    if (text == NULL) {
        fclose(in);
        llama3_fail("Memory allocation failed for buffer");
    }
    size_t have = 0;
    while (have < want) {
        const size_t n = fread(text + have, 1, want - have, in);
        if (n == 0) break;
        have += n;
    }
    fclose(in);
    text[have] = '\0';
    return text;
}

// ---- the byte trie -------------------------------------------------------------------------------------
// The node layout is the reference's (tokenizer.cuh:14-32: parallel arrays child_char / child_node, a capacity,
// a count, the id or -1).  What this file adds on top of that layout is an invariant: child_char is kept in
// ascending order of the bytes' unsigned values.  Look-ups are then binary searches, a whole vocabulary can be
// laid down from a sorted list in one pass with arrays of exactly the right size (bulk_build below), and a
// string added afterwards is spliced in at its place.

static inline unsigned char ub(char c) { return (unsigned char)c; }

// first slot whose byte is not below `c` (child_len when there is none)
static int child_slot(const TrieNode *node, char c) {
    int lo = 0, hi = node->child_len;
    while (lo < hi) {
        const int mid = (lo + hi) / 2;
        if (ub(node->child_char[mid]) < ub(c)) lo = mid + 1;
        else hi = mid;
    }
    return lo;
}

static TrieNode *new_node(int capacity) {
    TrieNode *node = (TrieNode *)malloc(sizeof(TrieNode));
    if (node == NULL) llama3_fail("Memory allocation failed for TrieNode");
    node->_max_childs = capacity > 0 ? capacity : 1;
    node->child_len = 0;
    node->token = -1;
    node->child_char = (char *)malloc(sizeof(char) * (size_t)node->_max_childs);
    node->child_node = (TrieNode **)malloc(sizeof(TrieNode *) * (size_t)node->_max_childs);
    if (node->child_char == NULL || node->child_node == NULL) llama3_fail("Memory allocation failed for child arrays");
    return node;
}

// tokenizer.cu:247-273: an empty node with room for one child
TrieNode *init_trienode() { return new_node(1); }

// tokenizer.cu:300-308: index of the child reached by byte `str` (and the child in *result), or -1
int _find_child(TrieNode *node, char str, TrieNode **result) {
    const int at = child_slot(node, str);
    if (at == node->child_len || node->child_char[at] != str) return -1;
    *result = node->child_node[at];
    return at;
}

// tokenizer.cu:310-332: twice the room for children
void _memexpand_child_nodes(TrieNode *node) {
    const int room = node->_max_childs * 2;
    char *bytes = (char *)realloc(node->child_char, sizeof(char) * (size_t)room);
    if (bytes == NULL) llama3_fail("Memory allocation failed during child_char expansion");
    node->child_char = bytes;
    TrieNode **kids = (TrieNode **)realloc(node->child_node, sizeof(TrieNode *) * (size_t)room);
    if (kids == NULL) llama3_fail("Memory allocation failed during child_node expansion");
    node->child_node = kids;
    node->_max_childs = room;
}

// tokenizer.cu:275-298: one string into an existing trie; a string that spells an existing path replaces its id.
// A missing child is spliced in at its sorted place.
void _build_trie(TrieNode *root, char *token_string, int token_int) {
    TrieNode *node = root;
    for (const char *p = token_string; *p != '\0'; ++p) {
        const int at = child_slot(node, *p);
        if (at < node->child_len && node->child_char[at] == *p) {
            node = node->child_node[at];
            continue;
        }
        if (node->child_len == node->_max_childs) _memexpand_child_nodes(node);
        const size_t behind = (size_t)(node->child_len - at);
        memmove(node->child_char + at + 1, node->child_char + at, behind * sizeof(char));
        memmove(node->child_node + at + 1, node->child_node + at, behind * sizeof(TrieNode *));
        TrieNode *fresh = init_trienode();
        node->child_char[at] = *p;
        node->child_node[at] = fresh;
        node->child_len += 1;
        node = fresh;
    }
    node->token = token_int;
}

} // extern "C"

// The whole vocabulary at once.  `entries` is sorted by string (bytes as unsigned values) with one entry per
// distinct string; entries[lo..hi) share their first `depth` bytes.  The strings that continue with the same
// next byte form a run; every run becomes one child, allocated with exactly as many slots as it has runs below.
namespace {
struct VocabEntry {
    std::string text; // up to the first NUL: the reference handles C strings (tokenizer.cu:279)
    int id;
    size_t order;     // position in the file: of two equal strings the later one's id stays (tokenizer.cu:83-96)
};

void bulk_build(TrieNode *node, const std::vector<VocabEntry> &entries, size_t lo, size_t hi, size_t depth) {
    if (lo < hi && entries[lo].text.size() == depth) { // the string that ends here sorts first
        node->token = entries[lo].id;
        ++lo;
    }
    int runs = 0;
    for (size_t i = lo; i < hi; ++i)
        if (i == lo || entries[i].text[depth] != entries[i - 1].text[depth]) ++runs;
    if (runs == 0) return;
    if (runs > node->_max_childs) {
        free(node->child_char);
        free(node->child_node);
        node->child_char = (char *)malloc(sizeof(char) * (size_t)runs);
        node->child_node = (TrieNode **)malloc(sizeof(TrieNode *) * (size_t)runs);
        if (node->child_char == NULL || node->child_node == NULL) llama3_fail("Memory allocation failed for child arrays");
        node->_max_childs = runs;
    }
    size_t begin = lo;
    while (begin < hi) {
        size_t end = begin + 1;
        while (end < hi && entries[end].text[depth] == entries[begin].text[depth]) ++end;
        TrieNode *child = new_node(1);
        node->child_char[node->child_len] = entries[begin].text[depth];
        node->child_node[node->child_len] = child;
        node->child_len += 1;
        bulk_build(child, entries, begin, end, depth + 1);
        begin = end;
    }
}

// sorts, drops all but the last-defined of equal strings, builds
void build_vocabulary(TrieNode *root, std::vector<VocabEntry> &entries) {
    std::sort(entries.begin(), entries.end(), [](const VocabEntry &a, const VocabEntry &b) {
        const int c = a.text.compare(b.text); // char_traits<char>::compare orders bytes as unsigned values
        return c != 0 ? c < 0 : a.order < b.order;
    });
    size_t kept = 0;
    for (size_t i = 0; i < entries.size(); ++i) {
        if (i + 1 < entries.size() && entries[i + 1].text == entries[i].text) continue; // a later definition follows
        if (kept != i) entries[kept] = std::move(entries[i]);
        ++kept;
    }
    entries.resize(kept);
    bulk_build(root, entries, 0, entries.size(), 0);
}
} // namespace

extern "C" {

// tokenizer.cu:334-343
static void build_decoder_entry(char **decoder, int decode_size, char *token_string, int token_int);
void _build_decoder(char **decoder, char *token_string, int token_int) {
    build_decoder_entry(decoder, g_decode_size, token_string, token_int);
}

static void build_decoder_entry(char **decoder, int decode_size, char *token_string, int token_int) {
    if (token_int < 0 || token_int >= decode_size)
        llama3_fail("token id %d is outside the decode table of %d entries", token_int, decode_size);
    free(decoder[token_int]);
    size_t length = strlen(token_string) + 1;
    decoder[token_int] = (char *)malloc(length);
    if (decoder[token_int] == NULL) llama3_fail("Memory allocation failed for decoder[%d].", token_int);
    memcpy(decoder[token_int], token_string, length);
}

Llama3Tokenizer *load_tokenizer_from(const char *filename, int decode_size) {
    if (decode_size < 1) llama3_fail("load_tokenizer_from: decode table size must be positive");
    g_decode_size = decode_size;
    Llama3Tokenizer *tok = (Llama3Tokenizer *)malloc(sizeof(Llama3Tokenizer));
    if (tok == NULL) llama3_fail("Memory allocation failed for Llama3 Tokenizer");
    tok->root = init_trienode();
    tok->decode = (char **)calloc((size_t)decode_size, sizeof(char *));
    if (tok->decode == NULL) llama3_fail("Memory allocation failed for the decode table");
    char *buffer = read_tokenizer_json(tok, filename);
    minijson::Value json;
    minijson::Parser parser(buffer, strlen(buffer));
    if (!parser.parse(json) || json.kind != minijson::Value::Object)
        llama3_fail("while parsing tokenizer.json structure");
    free(buffer);
    const minijson::Value *added = json.get("added_tokens");
    if (added == nullptr) llama3_fail("Could not find 'added_tokens' in the JSON");
    const minijson::Value *model = json.get("model");
    if (model == nullptr) llama3_fail("Could not find 'model' in the JSON");
    const minijson::Value *vocab = model->get("vocab");
    if (vocab == nullptr || vocab->kind != minijson::Value::Object)
        llama3_fail("Could not find 'vocab' in the model or it's not an object");
    // tokenizer.cu:83-96: vocabulary first, then the added (special) tokens.  The decode table takes every
    // definition in file order (a later one replaces an earlier one); the trie is laid down once from all of them.
    std::vector<VocabEntry> entries;
    entries.reserve(vocab->obj.size() + 64);
    auto define = [&](const std::string &text, int id) {
        std::string c_text(text.c_str()); // ends at the first NUL
        build_decoder_entry(tok->decode, decode_size, &c_text[0], id);
        entries.push_back(VocabEntry{std::move(c_text), id, entries.size()});
    };
    for (const auto &kv : vocab->obj) define(kv.first, (int)kv.second.num);
    if (added->kind == minijson::Value::Array) {
        for (const minijson::Value &e : added->arr) {
            const minijson::Value *id = e.get("id"), *content = e.get("content");
            if (id == nullptr || content == nullptr) continue;
            define(content->str, (int)id->num);
        }
    }
    build_vocabulary(tok->root, entries);
    return tok;
}

// tokenizer.cu:21-98
Llama3Tokenizer *load_tokenizer() { return load_tokenizer_from("model_weights/modified_tokenizer.json", 128256); }

// The longest vocabulary string that starts at `text` (at most `avail` bytes): its id and length, or -1.
// The walk ends at the first byte that has no child; the last node on the way that carried an id wins.
static int longest_match(TrieNode *const first_byte[256], const char *text, int avail, int *length) {
    int id = -1;
    TrieNode *node = first_byte[ub(text[0])];
    for (int used = 1; node != nullptr; ++used) {
        if (node->token != -1) {
            id = node->token;
            *length = used;
        }
        TrieNode *next = nullptr;
        if (used == avail || _find_child(node, text[used], &next) == -1) break;
        node = next;
    }
    return id;
}

// tokenizer.cu:100-155: tokens[0] = count + 1, ids in tokens[1..count], at most 2048 of them; from each
// position the longest vocabulary string that matches wins.  The root's children are spread into a table
// indexed by the first byte once per call, so every token starts with one indexed load.
int *tokenize(Llama3Tokenizer *tokenizer, char *input_str) {
    const int cap = 2048;
    int *tokens = (int *)malloc(sizeof(int) * (cap + 1));
    if (tokens == NULL) llama3_fail("Memory allocation failed for tokens");
    TrieNode *first_byte[256] = {nullptr};
    const TrieNode *root = tokenizer->root;
    for (int c = 0; c < root->child_len; ++c) first_byte[ub(root->child_char[c])] = root->child_node[c];
    const int total = (int)strlen(input_str);
    int count = 0;
    for (int at = 0; at < total && count < cap;) {
        int length = 0;
        const int id = longest_match(first_byte, input_str + at, total - at, &length);
        if (id == -1) llama3_fail("Unable to tokenize input at position %d", at);
        tokens[++count] = id;
        at += length;
    }
    tokens[0] = count + 1;
    return tokens;
}

static void free_trie(TrieNode *n) {
    if (n == nullptr) return;
    for (int i = 0; i < n->child_len; ++i) free_trie(n->child_node[i]);
    free(n->child_char);
    free(n->child_node);
    free(n);
}

void free_tokenizer(Llama3Tokenizer *tok, int decode_size) {
    if (tok == nullptr) return;
    free_trie(tok->root);
    for (int i = 0; i < decode_size; ++i) free(tok->decode[i]);
    free(tok->decode);
    free(tok);
}

// main.cu:26-59 without the terminal I/O: system prompt, user turn, assistant header
char *llama3_chat_prompt(const char *user_input) {
    static const char head[] =
        "<|begin_of_text|><|start_header_id|>system<|end_header_id|>\n\nAs a helpful assistant, answer the user "
        "questions in detail and accurately\n<|eot_id|><|start_header_id|>user<|end_header_id|>\n\n";
    static const char tail[] = "\n<|eot_id|><|start_header_id|>assistant<|end_header_id|>\n\n";
    size_t n = strlen(head) + strlen(user_input) + strlen(tail) + 1;
    char *out = (char *)malloc(n);
    if (out == NULL) llama3_fail("Failed to allocate memory");
    strcpy(out, head);
    strcat(out, user_input);
    strcat(out, tail);
    return out;
}

} // extern "C"
