// Tokenizers of the reference (tokenizer.js): a character-level table and GPT-2 byte-pair
// encoding, reading files instead of fetching them. The BPE vocabulary is rebuilt from the merges
// file alone when gpt_tokens.json is not at hand: ids 0..255 are the byte symbols in
// bytes_to_unicode order, id 256 + r is the concatenation of merge r, the last id is <|endoftext|>.
"use strict";
const fs = require("fs");

class Tokenizer {
  constructor() {
    this.encoder = undefined;
    this.decoder = undefined;
    this.vocab_size = undefined;
  }
  async load() { throw new Error("Not implemented."); }
  getVocabSize() { return this.vocab_size; }
  encode(str) { throw new Error("Not implemented."); }
  decode(arr) { throw new Error("Not implemented."); }
}

class SimpleTokenizer extends Tokenizer {
  // file: a {character: id} JSON (weights/tokenization/simple_tokens.json); or {chars: "..."} for
  // nanoGPT's table, the sorted set of characters
  async load(file) {
    if (file && typeof file === "object" && file.chars !== undefined) {
      this.encoder = {};
      Array.from(new Set(Array.from(file.chars))).sort().forEach((c, i) => { this.encoder[c] = i; });
    } else {
      this.encoder = JSON.parse(fs.readFileSync(file, "utf8"));
    }
    this.decoder = {};
    Object.keys(this.encoder).forEach((x) => { this.decoder[this.encoder[x]] = x; });
    this.vocab_size = Object.keys(this.encoder).length;
    return this;
  }
  encode(str) { return str.split("").map((x) => this.encoder[x]); }
  decode(arr) { return Array.from(arr).map((x) => this.decoder[x]).join(""); }
}

const range = (x, y) => {
  const res = [];
  for (let i = x; i < y; i++) res.push(i);
  return res;
};
const ord = (x) => x.charCodeAt(0);

const bytes_to_unicode = () => {
  const bs = range(ord("!"), ord("~") + 1).concat(range(ord("¡"), ord("¬") + 1), range(ord("®"), ord("ÿ") + 1));
  const cs = bs.slice();
  let n = 0;
  for (let b = 0; b < 256; b++) {
    if (!bs.includes(b)) {
      bs.push(b);
      cs.push(256 + n);
      n = n + 1;
    }
  }
  const result = {};
  bs.forEach((b, i) => { result[b] = String.fromCharCode(cs[i]); });
  return { map: result, order: cs.map((c) => String.fromCharCode(c)) };
};

const get_pairs = (word) => {
  const pairs = [];
  for (let i = 1; i < word.length; i++) pairs.push([word[i - 1], word[i]]);
  return pairs;
};

class GPT2Tokenizer extends Tokenizer {
  constructor() {
    super();
    this.pat = /'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+/gu;
  }

  async load(bpeFile, tokensFile) {
    const lines = fs.readFileSync(bpeFile, "utf8").split("\n");
    const bpe_merges = lines.slice(1).filter((x) => x.trim().length > 0).map((x) => x.split(/\s+/).filter((e) => e.length > 0));
    const { map, order } = bytes_to_unicode();
    this.byte_encoder = map;
    this.byte_decoder = {};
    Object.keys(map).forEach((b) => { this.byte_decoder[map[b]] = parseInt(b); });
    if (tokensFile) {
      this.encoder = JSON.parse(fs.readFileSync(tokensFile, "utf8"));
    } else {
      this.encoder = {};
      order.concat(bpe_merges.map((m) => m[0] + m[1]), ["<|endoftext|>"]).forEach((s, i) => { this.encoder[s] = i; });
    }
    this.decoder = {};
    Object.keys(this.encoder).forEach((x) => { this.decoder[this.encoder[x]] = x; });
    this.bpe_ranks = new Map(bpe_merges.map((m, i) => [m[0] + " " + m[1], i]));
    this.cache = new Map();
    this.vocab_size = Object.keys(this.encoder).length;
    return this;
  }

  encode(text) {
    if (!this.byte_encoder) throw new Error("Tokenizer not loaded.");
    let bpe_tokens = [];
    for (const m of text.matchAll(this.pat)) {
      const token = Array.from(Buffer.from(m[0], "utf8")).map((b) => this.byte_encoder[b]).join("");
      bpe_tokens = bpe_tokens.concat(this.bpe(token).split(" ").map((x) => this.encoder[x]));
    }
    return bpe_tokens;
  }

  decode(tokens) {
    if (!this.byte_decoder) throw new Error("Tokenizer not loaded.");
    const text = Array.from(tokens).map((x) => this.decoder[x]).join("");
    return Buffer.from(text.split("").map((x) => this.byte_decoder[x])).toString("utf8");
  }

  bpe(token) {
    if (this.cache.has(token)) return this.cache.get(token);
    let word = token.split("");
    let pairs = get_pairs(word);
    if (pairs.length === 0) return token;
    while (true) {
      // the pair with the lowest merge rank; pairs without a rank never win
      let best = null, bestRank = Infinity;
      for (const p of pairs) {
        const r = this.bpe_ranks.get(p[0] + " " + p[1]);
        if (r !== undefined && r < bestRank) { best = p; bestRank = r; }
      }
      if (best === null) break;
      const [first, second] = best;
      let new_word = [];
      let i = 0;
      while (i < word.length) {
        const j = word.indexOf(first, i);
        if (j === -1) {
          new_word = new_word.concat(word.slice(i));
          break;
        }
        new_word = new_word.concat(word.slice(i, j));
        i = j;
        if (word[i] === first && i < word.length - 1 && word[i + 1] === second) {
          new_word.push(first + second);
          i = i + 2;
        } else {
          new_word.push(word[i]);
          i = i + 1;
        }
      }
      word = new_word;
      if (word.length === 1) break;
      pairs = get_pairs(word);
    }
    const out = word.join(" ");
    this.cache.set(token, out);
    return out;
  }
}

module.exports = { Tokenizer, SimpleTokenizer, GPT2Tokenizer };
