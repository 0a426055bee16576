Binput_0JQQ>(%??oo#?vD?^7
?E!tw>^ܿs>Dth^ƴa?1g:L=&^\b+=S~[>uXr	t?