VERS_1.0 {
  global:
    plaidml_*;
  local:
    *;
};
