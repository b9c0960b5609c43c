// Prints, as JSON, what the JavaScript tokenizers make of the texts given on the command line:
// node tokenizer_checks.js <vocab.bpe> <text>...
"use strict";
const w = require("../../webgpt_amd/js/index.js");
async function main() {
  const t = await new w.GPT2Tokenizer().load(process.argv[2]);
  const out = { vocab_size: t.getVocabSize(), eot: t.encoder["<|endoftext|>"], ids: [], round: [] };
  for (const text of process.argv.slice(3)) {
    const ids = t.encode(text);
    out.ids.push(ids);
    out.round.push(t.decode(ids));
  }
  const s = await new w.SimpleTokenizer().load({ chars: "hello world" });
  out.simple = { ids: s.encode("low"), text: s.decode([3, 2, 2]), n: s.getVocabSize() };
  console.log(JSON.stringify(out));
}
main().catch((e) => { console.error(e); process.exit(1); });
