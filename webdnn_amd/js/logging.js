"use strict";
// Minimal leveled logger (no DOM).  Reference: src/descriptor_runner/logging.ts:65-246
// keeps a singleton on `window`; here it is a module-level object.
const LEVELS = { FATAL: 0, ERROR: 1, WARN: 2, INFO: 3, DEBUG: 4 };

const state = {
  level: LEVELS.WARN,
  // adapter(levelName, category, message, args)
  adapter: (levelName, category, message, args) => {
    const fn = levelName === "WARN" ? console.warn : levelName === "DEBUG" || levelName === "INFO" ? console.log : console.error;
    fn(`[${levelName}] ${category}: ${message}`, ...args);
  },
  records: null, // array when the in-memory adapter is on
};

function emit(levelName, category, message, args) {
  if (LEVELS[levelName] > state.level) return;
  if (state.records) state.records.push({ level: levelName, category, message, args });
  else state.adapter(levelName, category, message, args);
}

function getLogger(category) {
  return {
    fatal: (m, ...a) => emit("FATAL", category, m, a),
    error: (m, ...a) => emit("ERROR", category, m, a),
    warn: (m, ...a) => emit("WARN", category, m, a),
    info: (m, ...a) => emit("INFO", category, m, a),
    debug: (m, ...a) => emit("DEBUG", category, m, a),
  };
}

function setLevel(name) {
  if (!(name in LEVELS)) throw new Error(`Unknown log level ${name}`);
  state.level = LEVELS[name];
}

// Collect records in memory instead of printing (the reference's "file" adapter).
function captureToMemory(on) {
  state.records = on ? [] : null;
}

function takeRecords() {
  const r = state.records || [];
  if (state.records) state.records = [];
  return r;
}

module.exports = { getLogger, setLevel, captureToMemory, takeRecords, LEVELS };
