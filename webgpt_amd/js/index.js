// CommonJS entry point: the names the reference's <script> files put in the global scope.
"use strict";
module.exports = Object.assign({}, require("./globals.js"), require("./instructions.js"), require("./model.js"), require("./tokenizer.js"), require("./quantize.js"), { synth: require("./synth.js"), native: require("./native.js") });
