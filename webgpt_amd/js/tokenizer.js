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

// GPT-2's byte <-> printable-character table: the 188 bytes that print on their own ('!'..'~',
// '\u00a1'..'\u00ac', '\u00ae'..'\u00ff') stand for themselves, the other 68 are given the code points
// 256, 257, ... in ascending byte order. `order` lists the characters in the order the vocabulary
// numbers them (the printable ones first), `map` is byte -> character.
function byteSymbols() {
  const printable = (b) => (b >= 0x21 && b <= 0x7e) || (b >= 0xa1 && b <= 0xac) || (b >= 0xae && b <= 0xff);
  const map = {};
  const order = [];
  for (let b = 0; b < 256; b++) {
    if (printable(b)) {
      map[b] = String.fromCharCode(b);
      order.push(map[b]);
    }
  }
  let shifted = 0;
  for (let b = 0; b < 256; b++) {
    if (!printable(b)) {
      map[b] = String.fromCharCode(256 + shifted++);
      order.push(map[b]);
    }
  }
  return { map, order };
}

class GPT2Tokenizer extends Tokenizer {
  constructor() {
    super();
    this.pat = /'s|'t|'re|'ve|'m|'ll|'d| ?\p{L}+| ?\p{N}+| ?[^\s\p{L}\p{N}]+|\s+(?!\S)|\s+/gu;
  }

  async load(bpeFile, tokensFile) {
    const lines = fs.readFileSync(bpeFile, "utf8").split("\n");
    const bpe_merges = lines.slice(1).filter((x) => x.trim().length > 0).map((x) => x.split(/\s+/).filter((e) => e.length > 0));
    const { map, order } = byteSymbols();
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

  // Byte-pair merging of one pre-token: repeatedly the adjacent pair of symbols with the lowest
  // merge rank is joined, every occurrence of it in one left-to-right sweep (a joined symbol does not
  // take part in another join of the same sweep), until no adjacent pair has a rank.
  bpe(token) {
    const hit = this.cache.get(token);
    if (hit !== undefined) return hit;
    let symbols = Array.from(token);
    while (symbols.length > 1) {
      let rank = Infinity, at = -1;
      for (let i = 0; i + 1 < symbols.length; i++) {
        const r = this.bpe_ranks.get(symbols[i] + " " + symbols[i + 1]);
        if (r !== undefined && r < rank) { rank = r; at = i; }
      }
      if (at < 0) break;
      const left = symbols[at], right = symbols[at + 1];
      const merged = new Array(symbols.length);
      let n = 0;
      for (let i = 0; i < symbols.length; i++) {
        if (i + 1 < symbols.length && symbols[i] === left && symbols[i + 1] === right) {
          merged[n++] = left + right;
          i++;
        } else {
          merged[n++] = symbols[i];
        }
      }
      merged.length = n;
      symbols = merged;
    }
    const out = symbols.join(" ");
    this.cache.set(token, out);
    return out;
  }
}

module.exports = { Tokenizer, SimpleTokenizer, GPT2Tokenizer };
