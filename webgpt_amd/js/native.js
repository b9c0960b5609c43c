// Loads the N-API addon and points it at libwebgpt_amd.so. There is no fallback:
// a missing addon or library is an Error.
"use strict";
const path = require("path");
const fs = require("fs");

const addonPath = path.join(__dirname, "wgpt_addon.node");
if (!fs.existsSync(addonPath)) {
  throw new Error(`${addonPath} is missing: build it with \`make -C webgpt_amd/js\``);
}
const native = require(addonPath);
native.load(process.env.WEBGPT_AMD_LIB || path.join(__dirname, "..", "libwebgpt_amd.so"));
module.exports = native;
