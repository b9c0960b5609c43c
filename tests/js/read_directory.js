// Prints, as JSON, every tensor of a weight directory as the JavaScript loader hands it to the
// library (no GPU needed): {name: [values]}.
"use strict";
const fs = require("fs");
const path = require("path");
const w = require("../../webgpt_amd/js/index.js");

async function main() {
  const folder = process.argv[2];
  const gpt = new w.GPT(folder, "char");
  const params = await gpt.loadParameters(folder);
  const out = {};
  for (const name of gpt.directoryNames(params)) out[name] = Array.from(gpt.readTensor(folder, name, params));
  console.log(JSON.stringify(out));
}
main().catch((e) => { console.error(e); process.exit(1); });
