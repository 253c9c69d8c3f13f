
J%%ñ¾lÕÓ>`cœ¾Ð'X?ÒT¿Boutput_0