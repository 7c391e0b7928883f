// Host-side tokenizer of the llama2 extension: the sentencepiece-style BPE that the reference engine uses
// (CudaExtension.llm32.llama2/Files/llama2_tokenizer.cpp), restated on std containers.
//
// File format (build_tokenizer, llama2_tokenizer.cpp:28-52): int32 max_token_length, then per vocabulary entry
// float32 score, int32 byte length, the bytes.  The vocabulary size comes from the model configuration.
// encode (llama2_tokenizer.cpp:101-220): optional BOS (1); a " " dummy-prefix token when the text is not empty;
// one token per UTF-8 code point, or one token per byte (+3) when the code point is not in the vocabulary; then
// repeatedly merge the adjacent pair whose concatenation is the vocabulary entry with the highest score (the
// leftmost such pair on ties, strict '>') until no pair merges; optional EOS (2).
// decode (llama2_tokenizer.cpp:66-78): the entry's text, minus one leading space right after BOS; entries of the
// form <0xHH> stand for the raw byte.
#pragma once
#include <stdint.h>
#include <stdio.h>

#include <string>
#include <unordered_map>
#include <vector>

namespace mch {

class BpeTokenizer {
public:
    bool loaded() const { return !m_vocab.empty(); }
    int vocab_size() const { return (int)m_vocab.size(); }

    // returns false when the file is short or malformed
    bool load(const char* path, int vocabSize)
    {
        m_vocab.clear();
        m_scores.clear();
        m_index.clear();
        FILE* f = fopen(path, "rb");
        if (!f) return false;
        bool ok = vocabSize > 0 && fread(&m_maxTokenLength, sizeof(int32_t), 1, f) == 1;
        std::vector<std::string> vocab;
        std::vector<float> scores;
        for (int i = 0; ok && i < vocabSize; i++) {
            float score;
            int32_t len;
            ok = fread(&score, sizeof(float), 1, f) == 1 && fread(&len, sizeof(int32_t), 1, f) == 1 && len >= 0 && len < (1 << 20);
            if (!ok) break;
            std::string s((size_t)len, '\0');
            if (len > 0) ok = fread(&s[0], 1, (size_t)len, f) == (size_t)len;
            // the reference keeps C strings: anything after an embedded NUL is invisible to it
            s = std::string(s.c_str());
            vocab.push_back(s);
            scores.push_back(score);
        }
        fclose(f);
        if (!ok) return false;
        m_vocab.swap(vocab);
        m_scores.swap(scores);
        // exact-match lookup; the lowest id wins among duplicate strings
        for (int i = (int)m_vocab.size() - 1; i >= 0; i--) m_index[m_vocab[i]] = i;
        return true;
    }

    int lookup(const std::string& s) const
    {
        auto it = m_index.find(s);
        return it == m_index.end() ? -1 : it->second;
    }

    std::vector<int> encode(const std::string& textIn, bool bos, bool eos) const
    {
        const std::string text(textIn.c_str());   // stops at the first NUL, as the C string of the reference does
        std::vector<int> tokens;
        if (bos) tokens.push_back(1);
        if (!text.empty()) tokens.push_back(lookup(" "));   // -1 if the vocabulary has no " " entry, like the reference
        std::string cp;
        for (size_t i = 0; i < text.size(); i++) {
            const unsigned char c = (unsigned char)text[i];
            if ((c & 0xC0) != 0x80) cp.clear();            // not a continuation byte: a new code point starts
            cp.push_back((char)c);
            const unsigned char nx = i + 1 < text.size() ? (unsigned char)text[i + 1] : 0;
            if ((nx & 0xC0) == 0x80 && cp.size() < 4) continue;
            const int id = lookup(cp);
            if (id != -1) tokens.push_back(id);
            else
                for (unsigned char b : cp) tokens.push_back((int)b + 3);   // byte fallback: ids 3.. are the raw bytes
            cp.clear();
        }
        for (;;) {
            float best = -1e10f;
            int bestId = -1, bestIdx = -1;
            for (size_t i = 0; i + 1 < tokens.size(); i++) {
                const int id = lookup(piece(tokens[i]) + piece(tokens[i + 1]));
                if (id != -1 && m_scores[id] > best) {
                    best = m_scores[id];
                    bestId = id;
                    bestIdx = (int)i;
                }
            }
            if (bestIdx < 0) break;
            tokens[bestIdx] = bestId;
            tokens.erase(tokens.begin() + bestIdx + 1);
        }
        if (eos) tokens.push_back(2);
        return tokens;
    }

    std::string decode(int prevToken, int token) const
    {
        if (token < 0 || token >= (int)m_vocab.size()) return std::string();
        std::string p = m_vocab[token];
        if (prevToken == 1 && !p.empty() && p[0] == ' ') p.erase(0, 1);
        unsigned int byte = 0;
        // "<0x%02hhX>" of the reference: at most two hex digits are consumed after "<0x", nothing after them is checked
        if (p.size() >= 4 && p.compare(0, 3, "<0x") == 0 && sscanf(p.c_str() + 3, "%2X", &byte) == 1)
            return byte ? std::string(1, (char)(unsigned char)byte) : std::string();   // byte 0 is an empty C string there
        return p;
    }

private:
    const std::string& piece(int id) const
    {
        static const std::string empty;
        return id >= 0 && id < (int)m_vocab.size() ? m_vocab[id] : empty;
    }
    int32_t m_maxTokenLength = 0;
    std::vector<std::string> m_vocab;
    std::vector<float> m_scores;
    std::unordered_map<std::string, int> m_index;
};

}  // namespace mch
