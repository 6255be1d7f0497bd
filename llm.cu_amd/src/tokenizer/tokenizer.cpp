// Tokenizer of the reference (src/tokenizer/tokenizer.cu:21-155,200-343): a byte trie over the
// vocabulary of a Hugging Face tokenizer.json ("model"."vocab" and "added_tokens"), greedy longest
// match from the current byte, and a decode table id -> string.  Not BPE-merge exact, as in the
// reference.  The reference reads model_weights/modified_tokenizer.json (tokenizer.json with the byte
// markers for space and newline replaced, setup-tokenizer.py); load_tokenizer_from() takes the path and
// the table size instead.  Same structs, same names, same messages and exit(1) on failure; unlike the
// reference the decode table is zero-initialised, a missing "added_tokens" is reported as such, and
// nodes are released by free_tokenizer().
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>

#include "common/fail.h"
#include "llama3_host.h"
#include "safetensor/json.h"

// Size of the decode table that the reference-named _build_decoder() checks ids against (its signature
// carries no size).  Per thread, set by the load that is running on that thread; loads on different
// threads do not see each other's value.
static thread_local int g_decode_size = 128256;

extern "C" {

// tokenizer.cu:231-245
long _get_file_size(const char *filename) {
    FILE *file = fopen(filename, "rb");
    if (file == NULL) {
        perror("Failed to open file");
        return -1;
    }
    fseek(file, 0, SEEK_END);
    long size = ftell(file);
    fclose(file);
    return size;
}

// tokenizer.cu:200-229
char *read_tokenizer_json(Llama3Tokenizer *tokenizer, const char *filename) {
    (void)tokenizer;
    long size = _get_file_size(filename);
    if (size == -1) llama3_fail("Could not determine file size");
    char *buffer = (char *)malloc((size_t)size + 1);
    if (buffer == NULL) llama3_fail("Memory allocation failed for buffer");
    FILE *fp = fopen(filename, "r");
    if (fp == NULL) {
        free(buffer);
        llama3_fail("Could not open file %s", filename);
    }
    size_t got = fread(buffer, 1, (size_t)size, fp);
    buffer[got] = '\0';
    fclose(fp);
    return buffer;
}

// tokenizer.cu:247-273
TrieNode *init_trienode() {
    TrieNode *node = (TrieNode *)malloc(sizeof(TrieNode));
    if (node == NULL) llama3_fail("Memory allocation failed for TrieNode");
    node->_max_childs = 1;
    node->child_len = 0;
    node->token = -1;
    node->child_char = (char *)malloc(sizeof(char) * (size_t)node->_max_childs);
    node->child_node = (TrieNode **)malloc(sizeof(TrieNode *) * (size_t)node->_max_childs);
    if (node->child_char == NULL || node->child_node == NULL) llama3_fail("Memory allocation failed for child arrays");
    return node;
}

// tokenizer.cu:300-308
int _find_child(TrieNode *node, char str, TrieNode **result) {
    for (int i = 0; i < node->child_len; i++) {
        if (node->child_char[i] == str) {
            *result = node->child_node[i];
            return i;
        }
    }
    return -1;
}

// tokenizer.cu:310-332
void _memexpand_child_nodes(TrieNode *node) {
    node->_max_childs *= 2;
    char *cc = (char *)realloc(node->child_char, sizeof(char) * (size_t)node->_max_childs);
    if (cc == NULL) llama3_fail("Memory allocation failed during child_char expansion");
    node->child_char = cc;
    TrieNode **cn = (TrieNode **)realloc(node->child_node, sizeof(TrieNode *) * (size_t)node->_max_childs);
    if (cn == NULL) llama3_fail("Memory allocation failed during child_node expansion");
    node->child_node = cn;
}

// tokenizer.cu:275-298: a later string that spells an existing path replaces its id
void _build_trie(TrieNode *root, char *token_string, int token_int) {
    TrieNode *curr = root;
    for (char *ch = token_string; *ch != '\0'; ch++) {
        TrieNode *next;
        if (_find_child(curr, *ch, &next) == -1) {
            if (curr->child_len == curr->_max_childs) _memexpand_child_nodes(curr);
            curr->child_char[curr->child_len] = *ch;
            curr->child_node[curr->child_len] = init_trienode();
            curr->child_len += 1;
            curr = curr->child_node[curr->child_len - 1];
        } else {
            curr = next;
        }
    }
    curr->token = token_int;
}

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
    // tokenizer.cu:83-96: vocabulary first, then the added (special) tokens
    for (const auto &kv : vocab->obj) {
        std::string s = kv.first;
        _build_trie(tok->root, &s[0], (int)kv.second.num);
        build_decoder_entry(tok->decode, decode_size, &s[0], (int)kv.second.num);
    }
    if (added->kind == minijson::Value::Array) {
        for (const minijson::Value &e : added->arr) {
            const minijson::Value *id = e.get("id"), *content = e.get("content");
            if (id == nullptr || content == nullptr) continue;
            std::string s = content->str;
            _build_trie(tok->root, &s[0], (int)id->num);
            build_decoder_entry(tok->decode, decode_size, &s[0], (int)id->num);
        }
    }
    return tok;
}

// tokenizer.cu:21-98
Llama3Tokenizer *load_tokenizer() { return load_tokenizer_from("model_weights/modified_tokenizer.json", 128256); }

// tokenizer.cu:100-155: tokens[0] = count + 1, ids in tokens[1..count], at most 2048 of them; from each
// position the longest vocabulary string that matches wins
int *tokenize(Llama3Tokenizer *tokenizer, char *input_str) {
    const int max_tokens = 2048 + 1;
    int input_len = (int)strlen(input_str);
    int *tokens = (int *)malloc(sizeof(int) * max_tokens);
    if (tokens == NULL) llama3_fail("Memory allocation failed for tokens");
    int token_count = 0;
    int i = 0;
    while (i < input_len && token_count < 2048) {
        TrieNode *curr = tokenizer->root;
        int last_token = -1, last_token_len = 0;
        for (int j = i; j < input_len; j++) {
            TrieNode *next;
            if (_find_child(curr, input_str[j], &next) == -1) break;
            curr = next;
            if (curr->token != -1) {
                last_token = curr->token;
                last_token_len = j - i + 1;
            }
        }
        if (last_token == -1) llama3_fail("Unable to tokenize input at position %d", i);
        tokens[++token_count] = last_token;
        i += last_token_len;
    }
    tokens[0] = token_count + 1;
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
